"""The scheduler's decisions, with a stand-in for the forward pass: the next token of
a request is a function of the tokens it has so far, as a real model's greedy token
is, so that runs under different budgets and pool sizes can be compared."""

import pytest

from halite_amd.cache import CacheManager
from halite_amd.config import ServerConfig
from halite_amd.engine.scheduler import Request, Scheduler
from halite_amd.parts.base import PagedKVNeed
from halite_amd.sampling import SamplingParams


def next_token(ids):
    h = 17
    for t in ids:
        h = (h * 31 + t + 1) % 1009
    return h % 97


class FakeModel:
    """Checks what a real step function would check, and records the steps."""

    def __init__(self, cache):
        self.cache = cache
        self.plans = []

    def __call__(self, plan):
        spans, toks, lps, seen = [], [], [], set()
        for i, (r, k) in enumerate(plan.entries):
            assert r.slot is not None and r.slot not in seen and k >= 1
            seen.add(r.slot)
            assert self.cache.length(r.slot) == r.n_cached
            spans.append((r.slot, r.n_cached + k))
        self.cache.reserve(spans)  # must not raise: the scheduler checked
        for (slot, n) in spans:
            self.cache.advance(slot, n)
        for i, (r, k) in enumerate(plan.entries):
            if plan.wants_logits(i):
                toks.append(next_token(r.all_ids))
                lps.append(-0.5)
        self.plans.append([(r.id, k, plan.wants_logits(i)) for i, (r, k) in enumerate(plan.entries)])
        return toks, lps


def make(num_pages=65, page_size=4, n_slots=8, **conf):
    cache = CacheManager({0: PagedKVNeed(1, 8)}, page_size=page_size, num_pages=num_pages, n_slots=n_slots, allocate=False)
    model = FakeModel(cache)
    conf.setdefault("max_seqs_per_forward", n_slots)
    sched = Scheduler(cache, ServerConfig(page_size=page_size, **conf), model, context_len=512, stop_token_ids=())
    return sched, model, cache


def expected(prompt, n, stop=()):
    ids, out = list(prompt), []
    for _ in range(n):
        t = next_token(ids)
        out.append(t)
        ids.append(t)
        if t in stop:
            break
    return out


def prompts(lengths):
    return [[(7 * i + j) % 50 for j in range(n)] for i, n in enumerate(lengths)]


def test_everything_finishes_with_the_right_tokens():
    sched, model, cache = make(max_tokens_per_forward=16, chunked_prefill_size=8)
    ps = prompts([5, 17, 33, 64, 1, 2])
    for i, p in enumerate(ps):
        sched.add_request(Request(i, p, SamplingParams(max_new_tokens=12, ignore_eos=True)))
    done = sched.run_to_completion()
    assert sorted(r.id for r in done) == list(range(6))
    for r in done:
        assert r.output_ids == expected(ps[r.id], 12) and r.finished_reason.reason == "length"
        assert len(r.output_logprobs) == 12
    sched.check_idle()
    cache.check()
    # the budget holds in every step, and no prompt portion exceeds its limit
    for plan in model.plans:
        assert sum(k for _, k, _ in plan) <= 16
        assert all(k <= 8 for _, k, _ in plan)


def test_portions_and_wanted_rows():
    sched, model, _ = make(max_tokens_per_forward=10, chunked_prefill_size=6)
    sched.add_request(Request("a", list(range(20)), SamplingParams(max_new_tokens=3, ignore_eos=True)))
    sched.run_to_completion()
    # 20 prompt tokens in portions of 6: only the portion that ends the prompt wants logits
    assert model.plans[:4] == [[("a", 6, False)], [("a", 6, False)], [("a", 6, False)], [("a", 2, True)]]
    assert model.plans[4:] == [[("a", 1, True)], [("a", 1, True)]]


def test_decodes_ride_along_with_prompt_portions():
    sched, model, _ = make(max_tokens_per_forward=8, chunked_prefill_size=8)
    sched.add_request(Request("a", [1, 2, 3], SamplingParams(max_new_tokens=6, ignore_eos=True)))
    sched.step()
    sched.add_request(Request("b", list(range(30)), SamplingParams(max_new_tokens=2, ignore_eos=True)))
    sched.run_to_completion()
    mixed = [p for p in model.plans if len(p) == 2]
    assert mixed and all(p[0] == ("a", 1, True) and p[1][0] == "b" and p[1][1] == 7 for p in mixed[:2])


def test_first_come_first_served_and_slots():
    sched, model, _ = make(n_slots=2, max_tokens_per_forward=64)
    for i in range(5):
        sched.add_request(Request(i, [1, 2, 3, i], SamplingParams(max_new_tokens=4, ignore_eos=True)))
    done = sched.run_to_completion()
    first_seen = []
    for plan in model.plans:
        for rid, _, _ in plan:
            if rid not in first_seen:
                first_seen.append(rid)
        assert len(plan) <= 2
    assert first_seen == [0, 1, 2, 3, 4]
    assert len(done) == 5 and sched.stats.max_running == 2


def test_stop_tokens():
    p = prompts([9])[0]
    full = expected(p, 30)
    stop = full[4]
    sched, _, _ = make()
    sched.add_request(Request(0, p, SamplingParams(max_new_tokens=30, stop_token_ids=[stop])))
    sched.add_request(Request(1, p, SamplingParams(max_new_tokens=30, stop_token_ids=[stop], ignore_eos=True)))
    sched.add_request(Request(2, p, SamplingParams(max_new_tokens=0)))
    done = {r.id: r for r in sched.run_to_completion()}
    cut = full.index(stop) + 1
    assert done[0].output_ids == full[:cut] and done[0].finished_reason.reason == "stop"
    assert done[0].finished_reason.matched == stop  # the stop token is part of the output
    assert done[1].output_ids == full and done[1].finished_reason.reason == "length"
    assert done[2].output_ids == [] and done[2].finished_reason.reason == "length"
    # the engine-wide stop set (eos of the model) works the same way
    sched, _, _ = make()
    sched.stop_token_ids = {stop}
    sched.add_request(Request(0, p, SamplingParams(max_new_tokens=30)))
    assert sched.run_to_completion()[0].output_ids == full[:cut]


def test_pages_run_out_requests_are_retracted_and_outputs_do_not_change():
    ps = prompts([14, 9, 11, 6])
    want = [expected(p, 40) for p in ps]
    sched, model, cache = make(num_pages=31, max_tokens_per_forward=32, default_init_new_token_ratio=0.05)
    for i, p in enumerate(ps):
        sched.add_request(Request(i, p, SamplingParams(max_new_tokens=40, ignore_eos=True)))
    done = {r.id: r for r in sched.run_to_completion()}
    assert sched.stats.retractions > 0
    assert sum(r.n_retractions for r in done.values()) == sched.stats.retractions
    for i in range(4):
        assert done[i].output_ids == want[i]
    sched.check_idle()
    cache.check()
    assert 0 < sched.new_token_ratio <= 1.0


def test_retraction_takes_the_request_with_fewest_generated_tokens():
    sched, model, cache = make(num_pages=17, max_tokens_per_forward=32, default_init_new_token_ratio=0.01)
    sched.add_request(Request("old", list(range(8)), SamplingParams(max_new_tokens=30, ignore_eos=True)))
    for _ in range(6):
        sched.step()
    sched.add_request(Request("new", list(range(8)), SamplingParams(max_new_tokens=30, ignore_eos=True)))
    done = {r.id: r for r in sched.run_to_completion()}
    assert done["new"].n_retractions >= 1 and done["old"].n_retractions == 0
    assert done["new"].output_ids == expected(list(range(8)), 30)


def test_one_request_that_cannot_fit():
    sched, _, _ = make(num_pages=5)
    with pytest.raises(ValueError, match="can never fit"):
        sched.add_request(Request(0, list(range(10)), SamplingParams(max_new_tokens=20)))
    with pytest.raises(ValueError, match="context length"):
        sched.add_request(Request(0, list(range(500)), SamplingParams(max_new_tokens=20)))
    with pytest.raises(ValueError, match="empty prompt"):
        sched.add_request(Request(0, [], SamplingParams()))
    # pages taken by someone else: the single request left cannot go on
    sched, _, cache = make(num_pages=9)
    squatter = cache.admit()
    cache.reserve([(squatter, 24)])
    sched.add_request(Request(0, list(range(6)), SamplingParams(max_new_tokens=20, ignore_eos=True)))
    with pytest.raises(RuntimeError, match="No space left for only one request"):
        sched.run_to_completion()


def test_new_token_ratio_decays_and_resets():
    sched, _, _ = make(default_new_token_ratio_decay_steps=10)
    assert sched.new_token_ratio == pytest.approx(0.7)
    sched.add_request(Request(0, [1, 2, 3], SamplingParams(max_new_tokens=30, ignore_eos=True)))
    for _ in range(6):
        sched.step()
    assert sched.min_new_token_ratio <= sched.new_token_ratio < 0.7
    while sched.running or sched.waiting:
        sched.step()
    assert sched.new_token_ratio == pytest.approx(sched.min_new_token_ratio)
    assert sched.step() is None
    assert sched.new_token_ratio == pytest.approx(0.7)  # idle: back to the start


def test_admission_reserves_for_running_requests():
    # with ratio 1 a request is admitted only if its prompt and all its new tokens fit
    sched, model, _ = make(num_pages=21, default_init_new_token_ratio=1.0, max_tokens_per_forward=64)
    for i in range(3):
        sched.add_request(Request(i, list(range(10)), SamplingParams(max_new_tokens=30, ignore_eos=True)))
    done = sched.run_to_completion()
    assert len(done) == 3 and sched.stats.retractions == 0
    assert sched.stats.max_running == 2  # 2 * 40 tokens fit 80, the third waits


def test_requests_are_checked_before_they_wait_and_a_batch_can_be_dropped():
    sched, model, cache = make()
    sched.vocab_size = 97
    with pytest.raises(ValueError, match="outside the vocabulary of 97"):
        sched.add_request(Request("bad", [3, 97, 5], SamplingParams(max_new_tokens=4)))
    with pytest.raises(ValueError, match="outside the vocabulary"):
        sched.add_request(Request("neg", [3, -1], SamplingParams(max_new_tokens=4)))
    with pytest.raises(ValueError, match="empty prompt"):
        sched.add_request(Request("empty", [], SamplingParams(max_new_tokens=4)))
    assert not sched.waiting
    # a batch that is given up half way: slots and pages come back, the queues are empty
    for i in range(3):
        sched.add_request(Request(i, [1 + i] * (9 + i), SamplingParams(max_new_tokens=30, ignore_eos=True)))
    for _ in range(4):
        plan = sched.schedule()
        sched.process_results(plan, *model(plan))
    assert sched.running and not cache.idle()
    sched.abort_all()
    assert not sched.running and not sched.waiting and cache.idle()
    cache.check()
    sched.add_request(Request("next", [5, 6, 7], SamplingParams(max_new_tokens=6, ignore_eos=True)))
    while (plan := sched.schedule()) is not None:
        sched.process_results(plan, *model(plan))
    assert cache.idle()


class LetterTokenizer:
    """Token t is the letter chr(97 + t % 26)."""

    eos_id = None
    additional_stop_token_ids = None

    def encode(self, text, add_special_tokens=True):
        return [ord(c) - 97 for c in text]

    def decode(self, ids):
        return "".join(chr(97 + t % 26) for t in ids)


def test_stop_strings():
    """A request ends when the text of its last tokens holds one of its stop strings
    (src/halite/transformers/infer/engine/batch.py:206-215); the tokens that spell it
    are part of the output."""
    sched, model, cache = make()
    sched.tokenizer = tok = LetterTokenizer()
    p = [3, 1, 4, 1, 5]
    full = expected(p, 40)
    text = tok.decode(full)
    stop = text[6:9]  # three letters that the request will write
    first = text.index(stop) + len(stop)
    sched.add_request(Request(0, p, SamplingParams(max_new_tokens=40, stop=stop)))
    sched.add_request(Request(1, p, SamplingParams(max_new_tokens=40, stop=["zzzzzz", stop])))
    sched.add_request(Request(2, p, SamplingParams(max_new_tokens=40, stop="qqqqqqqq")))
    done = {r.id: r for r in sched.run_to_completion()}
    assert done[0].output_ids == full[:first] and done[0].finished_reason.reason == "stop"
    assert done[0].finished_reason.matched == stop
    assert done[1].output_ids == full[:first]
    assert done[2].output_ids == full and done[2].finished_reason.reason == "length"
    assert cache.idle()


def _tight_pool_run(retract_decode_steps):
    """16 short requests that together outgrow a pool of 399 one-token pages.  Returns the
    prompts, the scheduler, the finished requests and the number of steps that retracted."""
    ps = prompts([4 + i % 5 for i in range(16)])
    sched, model, cache = make(num_pages=400, page_size=1, n_slots=16, max_tokens_per_forward=256,
                               default_init_new_token_ratio=0.05, retract_decode_steps=retract_decode_steps)
    for i, p in enumerate(ps):
        sched.add_request(Request(i, p, SamplingParams(max_new_tokens=60, ignore_eos=True)))
    done, events, seen = {}, 0, 0
    while True:
        out = sched.step()
        if out is None:
            break
        done.update({r.id: r for r in out})
        if sched.stats.retractions != seen:
            events, seen = events + 1, sched.stats.retractions
    sched.check_idle()
    cache.check()
    return ps, sched, done, events


def test_retraction_leaves_headroom_so_that_the_next_steps_do_not_retract_again():
    # infer/engine/batch.py:478-481: requests give way until those that stay can decode
    # retract_decode_steps more tokens.  Making room for the step at hand only (which a
    # headroom of one step amounts to) has to retract again a step or two later, and the
    # request that went is run anew each time it is let in again.
    ps, sched, done, events = _tight_pool_run(20)
    _, short_sched, short_done, short_events = _tight_pool_run(1)
    for i, p in enumerate(ps):
        assert done[i].output_ids == expected(p, 60) == short_done[i].output_ids
    assert 0 < events <= 3, events
    assert short_events >= 3 * events
    assert sched.stats.retractions <= 12
    rerun = sched.stats.prefill_tokens - sum(len(p) for p in ps)
    short_rerun = short_sched.stats.prefill_tokens - sum(len(p) for p in ps)
    assert 0 < rerun < short_rerun
    assert rerun <= 320  # 302 as measured; one retraction per step re-runs 369


def test_a_model_without_paged_layers_is_limited_by_slots_only():
    from halite_amd.parts.base import StateNeed

    cache = CacheManager({}, {}, {0: {"mean": StateNeed((4,))}}, page_size=4, num_pages=2, n_slots=3, allocate=False)
    model = FakeModel(cache)
    sched = Scheduler(cache, ServerConfig(page_size=4, max_seqs_per_forward=3, max_tokens_per_forward=16,
                                          chunked_prefill_size=8), model, context_len=512)
    ps = prompts([30, 5, 17, 9, 2])
    for i, p in enumerate(ps):
        sched.add_request(Request(i, p, SamplingParams(max_new_tokens=10, ignore_eos=True)))
    done = {r.id: r for r in sched.run_to_completion()}
    assert len(done) == 5 and sched.stats.retractions == 0 and sched.stats.max_running == 3
    for i, p in enumerate(ps):
        assert done[i].output_ids == expected(p, 10)
    for plan in model.plans:
        assert sum(k for _, k, _ in plan) <= 16 and all(k <= 8 for _, k, _ in plan)
    sched.check_idle()
    cache.check()


def test_two_groups_one_with_a_window():
    # layers with all keys and layers with a window of 6 have pages of their own; the
    # group without a window is the one that runs out
    needs = {0: PagedKVNeed(1, 8), 1: PagedKVNeed(1, 8, window=6), 2: PagedKVNeed(1, 8)}
    ps = prompts([14, 9, 11, 6])
    want = [expected(p, 40) for p in ps]

    def run(num_pages):
        cache = CacheManager(needs, page_size=4, num_pages=num_pages, n_slots=8, allocate=False)
        assert len(cache.groups) == 2
        model = FakeModel(cache)
        sched = Scheduler(cache, ServerConfig(page_size=4, max_seqs_per_forward=8, max_tokens_per_forward=32,
                                              default_init_new_token_ratio=0.05), model, context_len=512)
        for i, p in enumerate(ps):
            sched.add_request(Request(i, p, SamplingParams(max_new_tokens=40, ignore_eos=True)))
        done = {r.id: r for r in sched.run_to_completion()}
        for i in range(4):
            assert done[i].output_ids == want[i]
        sched.check_idle()
        cache.check()
        return sched

    roomy = run(200)
    assert roomy.stats.retractions == 0 and roomy.stats.max_running == 4
    tight = run(31)
    assert tight.stats.retractions > 0
    # a request that the windowed group could hold but the other could not is refused
    cache = CacheManager(needs, page_size=4, num_pages=5, n_slots=8, allocate=False)
    sched = Scheduler(cache, ServerConfig(page_size=4), FakeModel(cache), context_len=512)
    with pytest.raises(ValueError, match="can never fit"):
        sched.add_request(Request(0, list(range(10)), SamplingParams(max_new_tokens=20)))
