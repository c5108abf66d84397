"""Schedules for replaying token sequences through the step function, as traces.

A trace is a list of steps ``{"step", "entries": [{"id", "tokens", "want"}], "end"}``,
the format ``bin/trace_run`` reads.  ``run_trace`` drives a ``ModelRunner`` in process
the way that program does; ``collect`` puts the logits back together per request.
"""

import random

from halite_amd.engine.batch import Segment


def whole(requests: dict) -> list:
    """Each request alone and whole, one step each."""
    return [
        {"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
        for i, (rid, toks) in enumerate(requests.items())
    ]


def tail_one_by_one(requests: dict, tail: int = 32) -> list:
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(len(toks) - tail, 0)
        cuts = ([head] if head else []) + [1] * (len(toks) - head)
        pos = 0
        for j, n in enumerate(cuts):
            last = pos + n == len(toks)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[pos : pos + n], "want": list(range(n))}],
                          "end": [rid] if last else []})
            pos += n
    return steps


def portions(requests: dict, sizes=(7, 2, 13, 3, 2, 29, 5, 2, 64, 11)) -> list:
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        pos, i = 0, 0
        while pos < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - pos)
            i += 1
            last = pos + n == len(toks)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[pos : pos + n], "want": list(range(n))}],
                          "end": [rid] if last else []})
            pos += n
    return steps


def mixed(requests: dict, seed: int = 0, max_live: int = 4, decode_tail: int = 12) -> list:
    """Up to ``max_live`` requests at a time: portions of some beside single tokens
    of others in the same step; some requests sit a step out; a request that ends
    makes room for the next, whose pages are the ones just given back."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}  # id -> position
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            toks = requests[rid]
            pos = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step
            left = len(toks) - pos
            n = 1 if left <= decode_tail else min(rng.choice([2, 3, 5, 8, 13, 21, 40]), left - decode_tail)
            want = list(range(n)) if rng.random() < 0.8 else ([n - 1] if rng.random() < 0.5 else [])
            entries.append({"id": rid, "tokens": toks[pos : pos + n], "want": want})
            live[rid] = pos + n
            if pos + n == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def peak_tokens(trace: list, page: int = 64) -> int:
    """The most tokens that live requests hold at any time, each rounded up to a
    multiple of ``page`` (what ``--max-tokens`` of the replay program means)."""
    held, peak = {}, 0
    for step in trace:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // page) * page for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def run_trace(runner, trace: list) -> dict:
    """Drives the runner as the replay program does; returns ``{step: logits}``."""
    slots, out = {}, {}
    for step in trace:
        segs = []
        for e in step["entries"]:
            if e["id"] not in slots:
                slots[e["id"]] = runner.admit()
            s = slots[e["id"]]
            segs.append(Segment(s, runner.cache.length(s), e["tokens"], list(e["want"])))
        logits = runner.step(segs)
        if logits.shape[0]:
            out[step["step"]] = logits.float().cpu()
        for rid in step["end"]:
            runner.free(slots.pop(rid))
        runner.cache.check()
    assert not slots
    return out


def collect(trace: list, step_logits: dict, vocab: int) -> dict:
    """``{request id: {position: logits row}}`` from per-step outputs."""
    pos, rows = {}, {}
    for step in trace:
        block = step_logits.get(step["step"])
        r = 0
        for e in step["entries"]:
            p0 = pos.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[p0 + w] = block[r]
                r += 1
            pos[e["id"]] = p0 + len(e["tokens"])
        assert block is None or r == block.shape[0]
    return rows


def compare(rows: dict, reference: dict, tol: float) -> float:
    """Largest error of any wanted row against the whole-sequence reference,
    relative to the largest logit (at least 1); asserts it is within ``tol``."""
    worst = 0.0
    for rid, by_pos in rows.items():
        ref = reference[rid]
        scale = max(1.0, float(ref.abs().max()))
        for p, row in by_pos.items():
            err = float((row - ref[p]).abs().max()) / scale
            assert err == err, f"request {rid} position {p}: NaN in the logits"
            if err > tol:
                bad = int((row - ref[p]).abs().argmax())
                raise AssertionError(
                    f"request {rid} position {p}: error {err:.3e} > {tol:.1e} "
                    f"(logit {bad}: {float(row[bad]):.6f} vs {float(ref[p][bad]):.6f})"
                )
            worst = max(worst, err)
    return worst
