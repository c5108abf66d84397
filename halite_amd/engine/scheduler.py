"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees; and decides what happens when pages run out.

Policy after the reference's ``infer`` engine: first-come admission under a budget of
cache tokens in which running requests count with ``new_token_ratio`` of what they may
still generate (src/halite/transformers/infer/engine/schedule_policy.py:12-112,
scheduler.py:211-289), the ratio's decay and reset (scheduler.py:32-45, 103, 284-287),
finishing by length or stop token (batch.py:180-204), and retraction when decoding runs
out of pages (batch.py:468-527): the request with the fewest generated tokens (ties: the
longest prompt) gives up its pages and goes back to the front of the queue with the
tokens it has generated, which are run again as part of its prompt.  Portions and the
mixed step are the ``tokainfer`` engine's
(src/halite/transformers/tokainfer/engine/scheduler.py:539-635): every step carries one
token of each decoding request and fills the rest of ``max_tokens_per_forward`` with
prompt portions, earlier requests first; only the portion that ends a prompt asks for
logits.

Three deliberate departures from the reference, each a fault there: results of every
step are collected (scheduler.py:66-75 drops the first step's), prompts are really cut
(schedule_policy.py:97-110 never does), and the ratio after a retraction is capped at 1
(batch.py:525 floors it at 1).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable

from ..cache import CacheManager
from ..config.engine import ServerConfig
from ..sampling.params import SamplingParams

CLIP_MAX_NEW_TOKENS = 4096  # schedule_policy.py:38, 82


@dataclass
class FinishReason:
    reason: str  # "length" | "stop"
    matched: int | str | None = None  # the stop token or the stop string
    length: int | None = None


class Request:
    """src/halite/transformers/infer/engine/batch.py:143-253"""

    def __init__(self, id, input_ids, sampling_params: SamplingParams | None = None, input_text=None):
        self.id = id
        self.input_ids = list(input_ids)
        self.input_text = input_text
        self.sampling_params = sampling_params or SamplingParams()
        self.output_ids: list[int] = []
        self.output_logprobs: list[float] = []
        self.finished_reason: FinishReason | None = None
        self.slot: int | None = None
        self.n_cached = 0  # tokens of input_ids + output_ids that are in the cache
        self.is_retracted = False
        self.n_retractions = 0
        self.seed = 0
        self._stop_window: int | None = None  # tokens of the longest stop string

    @property
    def all_ids(self) -> list[int]:
        return self.input_ids + self.output_ids

    def ids_between(self, start: int, end: int) -> list[int]:
        """``all_ids[start:end]`` without putting the two lists together."""
        n_in = len(self.input_ids)
        if end <= n_in:
            return self.input_ids[start:end]
        if start >= n_in:
            return self.output_ids[start - n_in : end - n_in]
        return self.input_ids[start:] + self.output_ids[: end - n_in]

    @property
    def n_total(self) -> int:
        return len(self.input_ids) + len(self.output_ids)

    @property
    def remaining(self) -> int:
        """Tokens that still have to be run before the next one can be sampled."""
        return self.n_total - self.n_cached

    @property
    def decoding(self) -> bool:
        return self.slot is not None and self.remaining == 1 and self.n_cached > 0

    def finished(self) -> bool:
        return self.finished_reason is not None

    def check_finished(self, stop_token_ids=(), tokenizer=None):
        """batch.py:180-215 of the reference: by length, by a stop token, by a stop string
        in the text of the last tokens (as many as the longest stop string has, and one)."""
        if self.finished():
            return
        p = self.sampling_params
        if len(self.output_ids) >= p.max_new_tokens:
            self.finished_reason = FinishReason("length", length=p.max_new_tokens)
            return
        last = self.output_ids[-1]
        if not p.ignore_eos and (last in p.stop_token_ids or last in stop_token_ids):
            self.finished_reason = FinishReason("stop", matched=last)
        if p.stop and tokenizer is not None:
            if self._stop_window is None:
                self._stop_window = max(len(_encode_plain(tokenizer, s)) for s in p.stop)
            tail = tokenizer.decode(self.output_ids[-(self._stop_window + 1):])
            for s in p.stop:
                if s in tail:
                    self.finished_reason = FinishReason("stop", matched=s)
                    return


def _encode_plain(tokenizer, text: str) -> list:
    try:
        return list(tokenizer.encode(text, add_special_tokens=False))
    except TypeError:
        return list(tokenizer.encode(text))


@dataclass
class StepPlan:
    entries: list[tuple[Request, int]]  # the request and how many of its next tokens run
    n_decode: int = 0
    n_prefill_tokens: int = 0

    def wants_logits(self, i: int) -> bool:
        r, k = self.entries[i]
        return r.n_cached + k == r.n_total


@dataclass
class SchedulerStats:
    steps: int = 0
    prefill_tokens: int = 0
    decode_tokens: int = 0
    retractions: int = 0
    finished: int = 0
    max_running: int = 0
    tokens_per_step: list[int] = field(default_factory=list)


# run_step(plan) -> (tokens, logprobs) for the entries that want logits, in order
RunStep = Callable[[StepPlan], tuple[list[int], list[float]]]


class Scheduler:
    def __init__(
        self,
        cache: CacheManager,
        server_config: ServerConfig,
        run_step: RunStep,
        context_len: int,
        stop_token_ids=(),
        vocab_size: int | None = None,
        tokenizer=None,
    ):
        self.tokenizer = tokenizer  # only for stop strings
        self.cache = cache
        self.conf = server_config
        self.run_step = run_step
        self.context_len = context_len
        self.vocab_size = vocab_size
        self.stop_token_ids = set(stop_token_ids)
        c = server_config
        self.init_new_token_ratio = min(c.default_init_new_token_ratio * c.schedule_conservativeness, 1.0)
        self.min_new_token_ratio = min(self.init_new_token_ratio * c.default_min_new_token_ratio_factor, 1.0)
        self.new_token_ratio_decay = (
            self.init_new_token_ratio - self.min_new_token_ratio
        ) / c.default_new_token_ratio_decay_steps
        self.initialize()

    def initialize(self):
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []  # admitted, in admission order
        self.new_token_ratio = self.init_new_token_ratio
        self.stats = SchedulerStats()

    # -- submission -----------------------------------------------------------------
    def check_request(self, req: Request) -> None:
        """Raises ``ValueError`` for a request that can never be served."""
        p = req.sampling_params
        if not req.input_ids:
            raise ValueError(f"request {req.id!r}: empty prompt")
        if self.vocab_size is not None:
            lo, hi = min(req.input_ids), max(req.input_ids)
            if lo < 0 or hi >= self.vocab_size:
                raise ValueError(
                    f"request {req.id!r}: token id {lo if lo < 0 else hi} outside the vocabulary of {self.vocab_size}"
                )
        longest = len(req.input_ids) + p.max_new_tokens
        if longest > self.context_len:
            raise ValueError(
                f"request {req.id!r}: prompt {len(req.input_ids)} + max_new_tokens "
                f"{p.max_new_tokens} exceeds the context length {self.context_len}"
            )
        # every group of pages must be able to hold the request when it is alone; a model
        # without paged layers has no such limit
        if any(g.pages_per_token_span(longest) > g.pool.capacity for g in self.cache.groups):
            raise ValueError(
                f"request {req.id!r}: {longest} tokens can never fit the cache pool of "
                f"{self.cache.token_capacity} tokens"
            )

    def add_request(self, req: Request) -> None:
        self.check_request(req)
        self.waiting.append(req)

    def abort_all(self) -> None:
        """Drops every request, waiting or running, and gives back what they hold (after
        an error in the middle of a batch)."""
        for req in self.running:
            if req.slot is not None:
                self.cache.free(req.slot)
                req.slot = None
        self.waiting.clear()
        self.running = []
        self.new_token_ratio = self.init_new_token_ratio

    # -- one step ---------------------------------------------------------------------
    def _fits(self, spans) -> bool:
        return self.cache.can_reserve(spans)

    def _max_portion(self, req: Request, spans, want: int) -> int:
        """The largest ``k <= want`` such that ``k`` more tokens of ``req`` fit
        beside the spans already planned."""
        if want <= 0:
            return 0
        if self._fits(spans + [(req.slot, req.n_cached + want)]):
            return want
        lo, hi = 0, want  # lo fits (0 tokens always do), hi does not
        while hi - lo > 1:
            mid = (lo + hi) // 2
            if self._fits(spans + [(req.slot, req.n_cached + mid)]):
                lo = mid
            else:
                hi = mid
        return lo

    def _retract(self, req: Request) -> None:
        self.cache.free(req.slot)
        self.running.remove(req)
        req.slot = None
        req.n_cached = 0
        req.is_retracted = True
        req.n_retractions += 1
        self.waiting.appendleft(req)
        self.stats.retractions += 1

    def _decoded_ahead(self, r: Request) -> int:
        """The length of a decoding request ``retract_decode_steps`` tokens on (or at its end,
        if that comes first)."""
        end = min(len(r.input_ids) + r.sampling_params.max_new_tokens, self.context_len)
        return max(r.n_cached + 1, min(r.n_cached + self.conf.retract_decode_steps, end))

    def _retraction_victim(self, candidates: list[Request]) -> Request:
        # batch.py:468-476: sorted by (generated, -prompt) descending, popped from the end
        return min(candidates, key=lambda r: (len(r.output_ids), -len(r.input_ids)))

    def _ratio_after_retraction(self) -> float:
        decoded = sum(len(r.output_ids) for r in self.running)
        budget = sum(r.sampling_params.max_new_tokens for r in self.running)
        if budget <= 0:
            return self.init_new_token_ratio
        est = (decoded + self.conf.retract_decode_steps * len(self.running)) / budget
        return min(1.0, est)

    def schedule(self) -> StepPlan | None:
        """Decides the next step; ``None`` when nothing is left to run."""
        if not self.running and not self.waiting:
            return None
        conf = self.conf

        # 1. one token for every decoding request; make room by retraction
        decoding = [r for r in self.running if r.decoding]
        retracted_any = False
        if decoding and not self._fits([(r.slot, r.n_cached + 1) for r in decoding]):
            # batch.py:468-527: requests give way until those that stay can all decode
            # ``retract_decode_steps`` more tokens, not just this one, so that the next steps
            # do not retract again (every retraction runs a whole prompt anew)
            while True:
                if len(self.running) == 1:
                    if not self._fits([(r.slot, r.n_cached + 1) for r in decoding]):
                        raise RuntimeError("No space left for only one request")
                    break
                victim = self._retraction_victim(self.running)
                self._retract(victim)
                retracted_any = True
                decoding = [r for r in decoding if r is not victim]
                if self._fits([(r.slot, self._decoded_ahead(r)) for r in decoding]):
                    break
        if retracted_any:
            self.new_token_ratio = self._ratio_after_retraction()
        elif decoding:
            self.new_token_ratio = max(self.new_token_ratio - self.new_token_ratio_decay, self.min_new_token_ratio)
        decoding = decoding[: conf.max_tokens_per_forward]
        entries: list[tuple[Request, int]] = [(r, 1) for r in decoding]
        spans = [(r.slot, r.n_cached + 1) for r in decoding]
        budget = min(conf.max_tokens_per_forward - len(entries), conf.max_prefill_tokens)
        n_prefill = 0

        # 2. portions of the prompts that are under way, earlier requests first
        in_step = {id(r) for r in decoding}
        for r in self.running:
            if budget <= 0:
                break
            if id(r) in in_step or r.decoding:
                continue
            k = self._max_portion(r, spans, min(r.remaining, conf.chunked_prefill_size, budget))
            if k > 0:
                entries.append((r, k))
                spans.append((r.slot, r.n_cached + k))
                budget -= k
                n_prefill += k

        # 3. admission, first come first served (scheduler.py:211-265)
        if not retracted_any and self.waiting and budget > 0:
            # One budget of cache tokens per group of pages (the reference has one pool):
            # what is free, less what the running requests are expected to take.  A group
            # with a window never holds more of a request than the window spans.  Without
            # any group (no paged layer) only the slots limit admission.
            groups = self.cache.groups
            remaining_total = [
                g.pool.available * g.page_size
                - sum(
                    g.tokens_held_at_most(
                        min(r.sampling_params.max_new_tokens - len(r.output_ids), CLIP_MAX_NEW_TOKENS)
                        * self.new_token_ratio
                        + (r.remaining if not r.decoding else 0)
                    )
                    for r in self.running
                )
                for g in groups
            ]
            while self.waiting and budget > 0 and self.cache.slots.available > 0:
                r = self.waiting[0]
                new_tokens = min(r.sampling_params.max_new_tokens - len(r.output_ids), CLIP_MAX_NEW_TOKENS)
                need = [g.tokens_held_at_most(r.n_total + new_tokens) for g in groups]
                if any(n > left for n, left in zip(need, remaining_total)) and self.running:
                    break  # AddRequestResult.NO_TOKEN
                r.slot = self.cache.admit()
                r.n_cached = 0
                k = self._max_portion(r, spans, min(r.remaining, conf.chunked_prefill_size, budget))
                if k <= 0:
                    self.cache.free(r.slot)
                    r.slot = None
                    break
                self.waiting.popleft()
                self.running.append(r)
                remaining_total = [left - n for left, n in zip(remaining_total, need)]
                entries.append((r, k))
                spans.append((r.slot, r.n_cached + k))
                budget -= k
                n_prefill += k

        if not entries:
            # nothing can move: pages are held by requests that cannot go on
            if len(self.running) <= 1:
                raise RuntimeError("No space left for only one request")
            self._retract(self._retraction_victim(self.running))
            self.new_token_ratio = self._ratio_after_retraction()
            return self.schedule()
        self.stats.max_running = max(self.stats.max_running, len(self.running))
        return StepPlan(entries, n_decode=len(decoding), n_prefill_tokens=n_prefill)

    def process_results(self, plan: StepPlan, tokens: list[int], logprobs: list[float]) -> list[Request]:
        """Advances the requests of a step that has run; returns those that finished.  A
        request that had finished before this step's results were read (the step was
        launched ahead) is passed over: its row is void."""
        finished = []
        j = 0
        for i, (r, k) in enumerate(plan.entries):
            if r.finished():
                j += 1  # only steps of one token each are launched ahead
                continue
            wants = plan.wants_logits(i)
            r.n_cached += k
            if not wants:
                continue
            tok, lp = tokens[j], logprobs[j]
            j += 1
            if r.sampling_params.max_new_tokens == 0:
                r.finished_reason = FinishReason("length", length=0)
            else:
                r.output_ids.append(int(tok))
                r.output_logprobs.append(float(lp))
                r.check_finished(self.stop_token_ids, self.tokenizer)
            if r.finished():
                self.cache.free(r.slot)
                r.slot = None
                self.running.remove(r)
                finished.append(r)
                self.stats.finished += 1
        self.stats.steps += 1
        self.stats.decode_tokens += plan.n_decode
        self.stats.prefill_tokens += plan.n_prefill_tokens
        self.stats.tokens_per_step.append(plan.n_decode + plan.n_prefill_tokens)
        return finished

    def step(self) -> list[Request] | None:
        """One scheduling decision and one forward; ``None`` when idle."""
        plan = self.schedule()
        if plan is None:
            # scheduler.py:101-103: idle resets the ratio; check_memory's invariant
            self.new_token_ratio = self.init_new_token_ratio
            return None
        tokens, logprobs = self.run_step(plan)
        return self.process_results(plan, tokens, logprobs)

    def run_to_completion(self) -> list[Request]:
        done = []
        while True:
            out = self.step()
            if out is None:
                return done
            done.extend(out)

    def check_idle(self) -> None:
        """The reference's ``check_memory`` (scheduler.py:109-123) as an assertion."""
        if not self.cache.idle():
            raise AssertionError("scheduler is idle but pages or slots are still held")
