"""The request and result types of the Python entry point
(src/halite/transformers/infer/types.py:9-64)."""

from __future__ import annotations

from typing import Any, NamedTuple


class InferenceRequest(NamedTuple):
    id: Any
    input_ids: list[int]
    sampling_params: Any  # SamplingParams or a dict of its fields


class InferenceResult:
    """One entry per sample of the request (``n`` of them).  The class restates the
    reference's result type (infer/types.py:15-64: the same fields, ``validate_lengths``
    and ``to_dict``), so that code written against that engine reads results unchanged."""

    def __init__(self, id, input_ids=None, output_ids=None, output_logprobs=None,
                 finish_reason=None, num_cached_prompt_tokens=None):
        self.id = id
        self.input_ids = [] if input_ids is None else input_ids
        self.output_ids = [] if output_ids is None else output_ids
        self.output_logprobs = [] if output_logprobs is None else output_logprobs
        self.finish_reason = [] if finish_reason is None else finish_reason
        self.num_cached_prompt_tokens = [] if num_cached_prompt_tokens is None else num_cached_prompt_tokens

    def validate_lengths(self):
        n = len(self.output_ids)
        if not (n == len(self.output_logprobs) == len(self.finish_reason) == len(self.num_cached_prompt_tokens)):
            raise ValueError("output_ids, output_logprobs, finish_reason and num_cached_prompt_tokens differ in length")

    def to_dict(self):
        return {
            "id": self.id,
            "input_ids": self.input_ids,
            "output_ids": self.output_ids,
            "output_logprobs": self.output_logprobs,
            "finish_reason": self.finish_reason,
        }

    def __repr__(self):
        return f"InferenceResult(id={self.id!r}, input_ids={self.input_ids}, output_ids={self.output_ids})"
