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


class _PinnedRing:
    """Pinned host buffers for results in flight, used in turn (at most two steps are
    in flight at a time)."""

    def __init__(self, n=4):
        self.bufs = [None] * n
        self.i = 0

    def take(self, words: int) -> torch.Tensor:
        self.i = (self.i + 1) % len(self.bufs)
        if self.bufs[self.i] is None or self.bufs[self.i].numel() < words:
            self.bufs[self.i] = torch.empty(max(2 * words, 1024), dtype=torch.int32, pin_memory=True)
        return self.bufs[self.i][:words]


class _InFlight:
    """A step on the GPU whose tokens are on their way to the host."""

    def __init__(self, plan: StepPlan, rows: list[Request], pinned: "_PinnedRing"):
        self.plan, self.rows, self._pinned = plan, rows, pinned
        self.row_of = {id(r): i for i, r in enumerate(rows)}
        self.tokens = None  # int32 on the device
        self._host = self._event = None

    def fetch(self, tokens: torch.Tensor, logprobs: torch.Tensor) -> None:
        self.tokens = tokens
        n = tokens.numel()
        # the two results are the halves of one buffer: one copy
        both = torch.as_strided(tokens, (2 * n,), (1,)) if tokens.data_ptr() + 4 * n == logprobs.data_ptr() else torch.cat((tokens, logprobs.view(torch.int32)))
        self._host = self._pinned.take(2 * n)
        self._host.copy_(both, non_blocking=True)
        self._event = torch.cuda.Event()
        self._event.record()

    def result(self) -> tuple[list[int], list[float]]:
        if self._host is None:
            return [], []
        self._event.synchronize()
        n = self._host.numel() // 2
        return self._host[:n].tolist(), self._host[n:].view(torch.float32).tolist()


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
        self._pinned = _PinnedRing()
        self.steps_launched_ahead = 0
        stop = set(getattr(getattr(model_runner, "config", None), "stop_token_ids", ()) or ())
        if tokenizer is not None:
            if getattr(tokenizer, "eos_id", None) is not None:
                stop.add(tokenizer.eos_id)
            stop.update(getattr(tokenizer, "additional_stop_token_ids", None) or ())
        self._stop_token_ids = stop
        self._new_scheduler()
        self.initialized = True

    def _new_scheduler(self):
        r = self.model_runner
        self.scheduler = Scheduler(
            r.cache, self.server_config, self._run_step, r.context_len, self._stop_token_ids,
            vocab_size=r.vocab_size, tokenizer=self.tokenizer,
        )

    @classmethod
    def from_pretrained(cls, folder: str, server_config: ServerConfig | None = None,
                        model_config: ModelConfig | None = None, tokenizer=None, seed: int = 0):
        return cls(ModelRunner.from_pretrained(folder, server_config, model_config), tokenizer, seed)

    # -- the step under the scheduler ------------------------------------------------
    def _launch(self, plan: StepPlan, before: "_InFlight | None" = None) -> "_InFlight":
        """Puts a step on the GPU and asks for its tokens; does not wait.  ``before`` is a
        step whose tokens have not been read yet: the requests of ``plan`` (one token
        each) are one position further than the scheduler knows, and take that token
        from ``before``'s result on the device."""
        segments, rows = [], []
        ahead = 0 if before is None else 1
        for i, (r, k) in enumerate(plan.entries):
            start = r.n_cached
            if before is not None:
                # the scheduler has not counted ``before`` yet; the cache has
                start = self.model_runner.cache.length(r.slot)
                ids, wants = [before.row_of[id(r)]], True  # the row of the token, not the token
            else:
                ids = r.ids_between(start, start + k)
                wants = plan.wants_logits(i)
            segments.append(Segment(r.slot, start, np.asarray(ids, dtype=np.int32), [k - 1] if wants else []))
            if wants:
                rows.append(r)
        logits = self.model_runner.step(segments, token_feed=None if before is None else before.tokens)
        flight = _InFlight(plan, rows, self._pinned)
        if rows:
            tokens, logprobs = self.sampler.forward(
                logits,
                [r.sampling_params for r in rows],
                [r.seed for r in rows],
                [len(r.output_ids) + ahead for r in rows],
            )
            flight.fetch(tokens, logprobs)
        return flight

    def _run_step(self, plan: StepPlan):
        return self._launch(plan).result()

    def _decode_again(self, flight: "_InFlight") -> StepPlan | None:
        """The step after ``flight`` if it can be told without ``flight``'s tokens: nothing
        waits, every running request gets a token from ``flight``, and those that do not
        end by length with it decode once more."""
        sched = self.scheduler
        if sched.waiting or len(flight.rows) != len(flight.plan.entries):
            return None
        if len(sched.running) != len(flight.rows) or any(r.slot is None for r in flight.rows):
            return None
        again = [
            r for r in flight.rows
            if not r.finished()
            and len(r.output_ids) + 1 < r.sampling_params.max_new_tokens
            and r.n_total + 2 <= self.model_runner.context_len
        ]
        if not again:
            return None
        return StepPlan([(r, 1) for r in again], n_decode=len(again))

    def _run(self) -> None:
        """Schedules and runs steps until nothing is left.  With
        ``scheduling_steps_ahead`` a decode step whose requests are known is launched
        before the tokens of the step before it are read."""
        from ..cache import NoSpace

        sched = self.scheduler
        ahead = self.server_config.scheduling_steps_ahead > 0
        flight = None
        while True:
            if flight is None:
                plan = sched.schedule()
                if plan is None:
                    sched.new_token_ratio = sched.init_new_token_ratio
                    return
                flight = self._launch(plan)
                if not ahead:
                    sched.process_results(plan, *flight.result())
                    flight = None
                continue
            nxt = self._decode_again(flight)
            following = None
            if nxt is not None:
                try:
                    following = self._launch(nxt, before=flight)
                    self.steps_launched_ahead += 1
                    sched.new_token_ratio = max(sched.new_token_ratio - sched.new_token_ratio_decay, sched.min_new_token_ratio)
                except NoSpace:
                    following = None  # the scheduler decides what gives way
            sched.process_results(flight.plan, *flight.result())
            flight = following

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
        if not self.initialized:
            raise RuntimeError("the engine was cleaned up; initialize() it and load weights first")
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
        for _, c in clones:  # all of them are looked at before the first is queued
            self.scheduler.check_request(c)
        try:
            for _, c in clones:
                self.scheduler.add_request(c)
            self._run()
        except BaseException:
            # nothing of a failed batch stays behind: the engine serves the next one
            self.scheduler.abort_all()
            raise
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

    def initialize(self, capture_graphs: bool = False):
        """After ``cleanup``: the cache pool and empty weight tensors are allocated again,
        and ``load_state_dict`` has to bring the weights before requests are served (the
        reference's engine is used the same way between the steps of a trainer,
        engine.py:33-52).  ``capture_graphs``: record the decode graphs of every batch
        size now (engine.py:33-41 does so) instead of at the first step of each size."""
        if self.model_runner.released:
            self.model_runner.restore()
            self._new_scheduler()
        if capture_graphs and self.model_runner.has_weights:
            self.model_runner.capture_graphs()
        self.initialized = True

    def load_state_dict(self, state_dict: dict, assign: bool = True):
        """New weights for the running engine (engine.py:48-52 of the reference; tensors
        are named as in a model folder and are always copied into the engine's own)."""
        self.model_runner.load_state_dict(state_dict)

    def cleanup(self):
        """Frees the cache pool, the captured graphs and the weights (engine.py:43-46 of
        the reference), so that something else can have the GPU's memory."""
        self.scheduler.abort_all()
        self.scheduler.initialize()
        self.model_runner.release()
        self.initialized = False
