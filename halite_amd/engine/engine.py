"""The Python entry point (src/halite/transformers/infer/engine/engine.py:13-106)."""

from __future__ import annotations

import time
from collections.abc import Sequence

import numpy as np
import torch

from ..config.engine import ModelConfig, ServerConfig
from ..sampling import Sampler, SamplingParams, request_seed
from .batch import Segment
from .runner import ModelRunner
from .scheduler import Request, Scheduler, StepPlan
from .types import InferenceRequest, InferenceResult


class InferenceEngine:
    """``InferenceEngine(model_runner, tokenizer).infer_batch(requests)``.

    The reference takes a built module, a tokenizer and two configuration objects
    (engine.py:14-31); here the module with its pools is the ``ModelRunner``, which
    ``from_pretrained`` builds from a model folder.  ``tokenizer`` may be ``None``
    when requests carry token ids; it needs ``encode`` and may have ``eos_id`` and
    ``additional_stop_token_ids`` (infer/engine/batch.py:197-201).
    """

    def __init__(self, model_runner: ModelRunner, tokenizer=None, seed: int = 0):
        self.model_runner = model_runner
        self.tokenizer = tokenizer
        self.server_config = model_runner.server_config
        self.model_config = model_runner.model_config
        self.seed = seed
        self.sampler = Sampler(model_runner.device)
        stop = set(getattr(getattr(model_runner, "config", None), "stop_token_ids", ()) or ())
        if tokenizer is not None:
            if getattr(tokenizer, "eos_id", None) is not None:
                stop.add(tokenizer.eos_id)
            stop.update(getattr(tokenizer, "additional_stop_token_ids", None) or ())
        self.scheduler = Scheduler(
            model_runner.cache, self.server_config, self._run_step, model_runner.context_len, stop
        )
        self.initialized = True

    @classmethod
    def from_pretrained(cls, folder: str, server_config: ServerConfig | None = None,
                        model_config: ModelConfig | None = None, tokenizer=None, seed: int = 0):
        return cls(ModelRunner.from_pretrained(folder, server_config, model_config), tokenizer, seed)

    # -- the step under the scheduler ------------------------------------------------
    def _run_step(self, plan: StepPlan):
        segments, rows = [], []
        for i, (r, k) in enumerate(plan.entries):
            ids = r.ids_between(r.n_cached, r.n_cached + k)
            wants = plan.wants_logits(i)
            segments.append(Segment(r.slot, r.n_cached, np.asarray(ids, dtype=np.int32), [k - 1] if wants else []))
            if wants:
                rows.append(r)
        logits = self.model_runner.step(segments)
        if not rows:
            return [], []
        tokens, logprobs = self.sampler.forward(
            logits,
            [r.sampling_params for r in rows],
            [r.seed for r in rows],
            [len(r.output_ids) for r in rows],
        )
        # the two results are the halves of one buffer: one copy, one wait
        n = tokens.numel()
        if tokens.data_ptr() + 4 * n == logprobs.data_ptr():
            host = torch.as_strided(tokens, (2 * n,), (1,)).cpu()
            return host[:n].tolist(), host[n:].view(torch.float32).tolist()
        return tokens.tolist(), logprobs.tolist()

    # -- requests ----------------------------------------------------------------------
    def build_batch_request(self, requests) -> list[Request]:
        """Accepts the reference's request forms (scheduler.py:125-168): a string, an
        ``InferenceRequest``, ``(text_or_ids, params)``, ``(id, text_or_ids, params)``
        or a ``Request``; parameters may be a dict."""
        out = []
        for i, req in enumerate(requests):
            if isinstance(req, str):
                req = Request(i, self._encode(req), SamplingParams(), req)
            elif isinstance(req, InferenceRequest):
                req = Request(req.id, req.input_ids, self._params(req.sampling_params))
            elif isinstance(req, Request):
                pass
            elif isinstance(req, Sequence):
                if len(req) == 2:
                    id, (text_or_ids, params) = i, req
                elif len(req) == 3:
                    id, text_or_ids, params = req
                else:
                    raise ValueError(f"invalid request: {req!r}")
                text = text_or_ids if isinstance(text_or_ids, str) else None
                ids = self._encode(text_or_ids) if text is not None else list(text_or_ids)
                req = Request(id, ids, self._params(params), text)
            else:
                raise ValueError(f"Invalid request type: {type(req)}")
            if req.sampling_params.stop and self.tokenizer is None:
                raise ValueError("stop strings need a tokenizer")
            out.append(req)
        return out

    def _encode(self, text: str) -> list[int]:
        if self.tokenizer is None:
            raise ValueError("a text request needs a tokenizer; pass token ids instead")
        return list(self.tokenizer.encode(text))

    @staticmethod
    def _params(p) -> SamplingParams:
        if isinstance(p, SamplingParams):
            return p
        return SamplingParams(**(p or {}))

    def infer_batch(self, requests) -> list[InferenceResult]:
        requests = self.build_batch_request(requests)
        if not requests:
            return []
        n = requests[0].sampling_params.n
        if any(r.sampling_params.n != n for r in requests):
            raise ValueError("all requests must have the same number of samples")
        t0 = time.perf_counter()
        clones: list[tuple[Request, Request]] = []
        for req in requests:
            for j in range(n):
                c = Request((req.id, j), req.input_ids, req.sampling_params, req.input_text)
                c.seed = request_seed(req.sampling_params, req.id, self.seed) + j
                clones.append((req, c))
                self.scheduler.add_request(c)
        self.scheduler.run_to_completion()
        self.scheduler.check_idle()
        self.last_elapsed = time.perf_counter() - t0
        by_id: dict = {}
        order = []
        for req, c in clones:
            if id(req) not in by_id:
                by_id[id(req)] = InferenceResult(req.id, req.input_ids)
                order.append(by_id[id(req)])
            res = by_id[id(req)]
            res.output_ids.append(c.output_ids)
            res.output_logprobs.append(c.output_logprobs)
            res.finish_reason.append(c.finished_reason.reason)
            res.num_cached_prompt_tokens.append(0)
        try:
            return sorted(order, key=lambda r: r.id)
        except TypeError:
            return order

    @property
    def stats(self):
        return self.scheduler.stats

    def initialize(self):
        self.initialized = True

    def load_state_dict(self, state_dict: dict, assign: bool = True):
        """New weights for the running engine (engine.py:48-52 of the reference; tensors
        are named as in a model folder and are always copied into the engine's own)."""
        self.model_runner.load_state_dict(state_dict)

    def cleanup(self):
        self.scheduler.initialize()
        self.initialized = False
