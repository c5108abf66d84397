"""Generation through the entry point and the command line, against the plain
implementation."""

import json
import os
import subprocess
import sys

import pytest
import torch

import plain_llama
import tiny
from halite_amd.config import ModelConfig, ServerConfig
from halite_amd.engine import InferenceEngine, InferenceRequest
from halite_amd.sampling import SamplingParams, request_seed

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("A", tiny.TINY_A), ("B", tiny.TINY_B)):
        w = tiny.random_weights(cfg, seed=21, std=0.08)
        for dtype, store in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
            folder = str(tmp_path_factory.mktemp(f"gen{name}{dtype}"))
            tiny.write_model_folder(folder, cfg, w, store)
            out[(name, dtype)] = (folder, *plain_llama.read_model_folder(folder))
    return out


def check_against_plain(pc, pw, prompt, got, params, gap_limit, margin_limit):
    """Teacher-forced on the engine's own tokens: at every step the plain model's
    choice must be the engine's, unless the decision is closer than rounding."""
    ids = list(prompt)
    for step, tok in enumerate(got):
        logits = plain_llama.forward(pc, pw, ids)[-1]
        want, _, margin = plain_llama.sample_token(logits, params, step)
        if tok != want:
            if margin is None:
                assert float(logits[want] - logits[tok]) <= gap_limit, f"token {step}: engine {tok}, plain {want}"
            else:
                assert margin <= margin_limit, f"token {step}: engine {tok}, plain {want} (margin {margin})"
        ids.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation(models, dtype):
    folder, pc, pw = models[("A", dtype)]
    engine = InferenceEngine.from_pretrained(folder, ServerConfig(kv_cache_num_tokens=1024), ModelConfig(dtype=dtype))
    prompts = [tiny.random_tokens(tiny.TINY_A, n, 40 + n) for n in (5, 17, 33, 64)]
    params = {"max_new_tokens": 16, "temperature": 0.0}
    results = engine.infer_batch([InferenceRequest(f"q{i}", p, params) for i, p in enumerate(prompts)])
    assert [r.id for r in results] == ["q0", "q1", "q2", "q3"]
    for r, p in zip(results, prompts):
        assert r.input_ids == p and len(r.output_ids) == 1 and len(r.output_ids[0]) == 16
        assert r.finish_reason == ["length"] and len(r.output_logprobs[0]) == 16
        check_against_plain(pc, pw, p, r.output_ids[0], params, 1e-4 if dtype == "float32" else 0.06, 0)
        if dtype == "float32":
            want, lps, _ = plain_llama.generate(pc, pw, p, params)
            assert r.output_ids[0] == want
            assert max(abs(a - b) for a, b in zip(r.output_logprobs[0], lps)) < 1e-4
    # top_k = 1 asks for the same thing, whatever the temperature
    again = engine.infer_batch([(p, {"max_new_tokens": 16, "top_k": 1, "temperature": 0.7}) for p in prompts])
    assert [r.output_ids for r in again] == [r.output_ids for r in results]
    assert engine.model_runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_sampling_with_a_seed(models, dtype):
    folder, pc, pw = models[("B", dtype)]
    engine = InferenceEngine.from_pretrained(folder, ServerConfig(kv_cache_num_tokens=1024, page_size=16), ModelConfig(dtype=dtype))
    prompts = [tiny.random_tokens(tiny.TINY_B, n, 50 + n) for n in (1, 40, 100)]
    params = SamplingParams(max_new_tokens=24, temperature=0.8, seed=1234)
    results = engine.infer_batch([(i, p, params) for i, p in enumerate(prompts)])
    plain_params = {"temperature": 0.8, "seed": request_seed(params, 0), "max_new_tokens": 24}
    for r, p in zip(results, prompts):
        assert len(r.output_ids[0]) == 24
        check_against_plain(pc, pw, p, r.output_ids[0], plain_params, 0, 2e-4 if dtype == "float32" else 2e-2)
    # the same seed gives the same tokens, alone or beside other requests
    # (bfloat16 logits move by rounding with the batch, which can flip a draw that
    # falls next to an interval's edge, so the strict comparison is the 32-bit one)
    alone = engine.infer_batch([(7, prompts[1], params)])
    if dtype == "float32":
        assert alone[0].output_ids == results[1].output_ids
    else:
        # every token of the run alone is the plain implementation's draw from the same stream,
        # or a draw within rounding of an interval's edge; and up to the first such draw the two
        # runs are the same tokens
        check_against_plain(pc, pw, prompts[1], alone[0].output_ids[0], plain_params, 0, 2e-2)
        a, b = alone[0].output_ids[0], results[1].output_ids[0]
        same = next((i for i in range(24) if a[i] != b[i]), 24)
        assert same >= 4
        if same < 24:
            logits = plain_llama.forward(pc, pw, prompts[1] + a[:same])[-1]
            _, _, margin = plain_llama.sample_token(logits, plain_params, same)
            assert margin is not None and margin <= 2e-2, (same, margin)
    other = engine.infer_batch([(0, prompts[1], SamplingParams(max_new_tokens=24, temperature=0.8, seed=99))])
    assert other[0].output_ids != results[1].output_ids
    # n samples of one request draw from different streams
    many = engine.infer_batch([(0, prompts[1], SamplingParams(max_new_tokens=12, temperature=1.0, seed=5, n=3))])
    assert len(many[0].output_ids) == 3 and len({tuple(o) for o in many[0].output_ids}) == 3


def test_filters_and_stop_tokens_through_the_engine(models):
    folder, pc, pw = models[("A", "float32")]
    engine = InferenceEngine.from_pretrained(folder, ServerConfig(kv_cache_num_tokens=512), ModelConfig(dtype="float32"))
    p = tiny.random_tokens(tiny.TINY_A, 20, 3)
    params = SamplingParams(max_new_tokens=12, temperature=1.3, top_k=7, top_p=0.9, seed=8)
    r = engine.infer_batch([(0, p, params)])[0]
    plain_params = {"temperature": 1.3, "top_k": 7, "top_p": 0.9, "seed": 8}
    check_against_plain(pc, pw, p, r.output_ids[0], plain_params, 0, 2e-4)
    greedy, _, _ = plain_llama.generate(pc, pw, p, {"temperature": 0.0, "max_new_tokens": 12})
    stop = greedy[5]
    r = engine.infer_batch([(0, p, {"temperature": 0.0, "max_new_tokens": 12, "stop_token_ids": [stop]})])[0]
    assert r.output_ids[0] == greedy[: greedy.index(stop) + 1] and r.finish_reason == ["stop"]
    with pytest.raises(ValueError, match="tokenizer"):
        engine.infer_batch(["some text"])


def test_portions_retraction_and_page_reuse_keep_the_tokens(models):
    """Greedy output does not depend on the budget, on the portions, or on requests
    being thrown out and run again when pages run out."""
    folder, pc, pw = models[("A", "float32")]
    prompts = [tiny.random_tokens(tiny.TINY_A, n, 60 + n) for n in (30, 9, 41, 17, 25, 12)]
    params = {"max_new_tokens": 40, "temperature": 0.0, "ignore_eos": True}
    roomy = InferenceEngine.from_pretrained(folder, ServerConfig(kv_cache_num_tokens=2048, page_size=16), ModelConfig(dtype="float32"))
    want = [r.output_ids[0] for r in roomy.infer_batch([(i, p, params) for i, p in enumerate(prompts)])]
    tight = InferenceEngine.from_pretrained(
        folder,
        ServerConfig(kv_cache_num_tokens=160, page_size=16, max_tokens_per_forward=24, chunked_prefill_size=11,
                     default_init_new_token_ratio=0.05),
        ModelConfig(dtype="float32"),
    )
    got = tight.infer_batch([(i, p, params) for i, p in enumerate(prompts)])
    # requests are thrown out, but with headroom: a handful of times, not once a step
    assert 0 < tight.stats.retractions <= 8, tight.stats.retractions
    rerun = tight.stats.prefill_tokens - sum(len(p) for p in prompts)
    assert rerun <= 4 * sum(len(p) + 40 for p in prompts) // 3
    assert max(tight.stats.tokens_per_step) <= 24
    assert [r.output_ids[0] for r in got] == want
    assert tight.model_runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graph", [False, True])
def test_steps_launched_ahead_give_the_same_tokens(models, dtype, graph):
    """``scheduling_steps_ahead=1``: decode steps are launched before the tokens of the
    step before them are read.  Lengths that differ, stop tokens that end requests at
    unknown steps (their next row is void), sampling with seeds, requests that wait for a
    slot: the outputs equal those of the engine that waits for every step."""
    folder, pc, pw = models[("B", dtype)]
    prompts = [tiny.random_tokens(tiny.TINY_B, n, 300 + n) for n in (3, 40, 17, 64, 9, 30)]
    plain = InferenceEngine.from_pretrained(
        folder, ServerConfig(kv_cache_num_tokens=2048, max_seqs_per_forward=4, use_cudagraph=graph), ModelConfig(dtype=dtype))
    ahead = InferenceEngine.from_pretrained(
        folder, ServerConfig(kv_cache_num_tokens=2048, max_seqs_per_forward=4, use_cudagraph=graph, scheduling_steps_ahead=1),
        ModelConfig(dtype=dtype))
    # greedy with stop tokens taken from what the model really generates, so that requests end early
    free_run = plain.infer_batch([(p, {"max_new_tokens": 24, "temperature": 0.0}) for p in prompts])
    stops = {r.output_ids[0][5 + i] for i, r in enumerate(free_run)}
    for params in (
        [{"max_new_tokens": 5 + 3 * i, "temperature": 0.0} for i in range(6)],
        [{"max_new_tokens": 24, "temperature": 0.0, "stop_token_ids": sorted(stops)} for _ in range(6)],
        [{"max_new_tokens": 12, "temperature": 0.9, "top_p": 0.8, "seed": 11 + i} for i in range(6)],
        [{"max_new_tokens": 1 if i % 2 else 7, "temperature": 0.0} for i in range(6)],
    ):
        want = plain.infer_batch(list(zip(prompts, params)))
        got = ahead.infer_batch(list(zip(prompts, params)))
        if dtype == "float32" or params[0]["temperature"] == 0.0:
            assert [r.output_ids for r in got] == [r.output_ids for r in want]
            assert [r.finish_reason for r in got] == [r.finish_reason for r in want]
        for a, b in zip(got, want):
            assert len(a.output_ids[0]) == len(a.output_logprobs[0])
            if a.output_ids == b.output_ids:
                assert max(abs(x - y) for x, y in zip(a.output_logprobs[0], b.output_logprobs[0])) < 1e-5
        if "stop_token_ids" in params[0]:
            assert sum(r.finish_reason == ["stop"] for r in want) >= 3
        assert ahead.model_runner.cache.idle() and plain.model_runner.cache.idle()
    # some steps really were launched ahead
    assert ahead.steps_launched_ahead > 10 and plain.steps_launched_ahead == 0


def test_new_weights_for_a_running_engine(models, tmp_path):
    """``load_state_dict`` takes tensors named as in a model folder: afterwards the
    engine generates what an engine built from those weights generates (graphs that were
    captured with the old tensors included), and a bad dict is refused with the list."""
    from halite_amd.weights import WeightError

    folder, pc, pw = models[("A", "float32")]
    server = ServerConfig(kv_cache_num_tokens=1024, use_cudagraph=True)
    engine = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="float32"))
    prompt = tiny.random_tokens(tiny.TINY_A, 20, 7)
    params = {"max_new_tokens": 12, "temperature": 0.0}
    before = engine.infer_batch([(prompt, params)])[0].output_ids[0]
    other = tiny.random_weights(tiny.TINY_A, seed=99, std=0.08)
    engine.load_state_dict(other)
    after = engine.infer_batch([(prompt, params)])[0].output_ids[0]
    new_folder = str(tmp_path / "other")
    tiny.write_model_folder(new_folder, tiny.TINY_A, other, torch.float32)
    fresh = InferenceEngine.from_pretrained(new_folder, server, ModelConfig(dtype="float32"))
    assert after == fresh.infer_batch([(prompt, params)])[0].output_ids[0] and after != before
    broken = dict(other)
    broken.pop("model.norm.weight")
    broken["extra.weight"] = torch.zeros(3)
    with pytest.raises(WeightError, match="model.norm.weight") as err:
        engine.load_state_dict(broken)
    assert "extra.weight" in str(err.value)


def test_cleanup_gives_the_memory_back_and_initialize_brings_the_engine_back(models):
    """``cleanup`` frees pool, graphs and weights (a second engine of the same size fits in
    what came back); ``initialize`` and ``load_state_dict`` make the first one serve again,
    with the same tokens."""
    folder, pc, pw = models[("B", "bfloat16")]
    server = ServerConfig(kv_cache_num_tokens=65536, use_cudagraph=True)
    prompt = tiny.random_tokens(tiny.TINY_B, 20, 7)
    params = {"max_new_tokens": 12, "temperature": 0.0}
    import gc

    gc.collect()  # what earlier tests left behind must not go away in the middle of the count
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    engine = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="bfloat16"))
    before = engine.infer_batch([(prompt, params)])[0].output_ids[0]
    held = torch.cuda.memory_allocated() - base
    pool = engine.model_runner.cache.groups[0].storage
    assert held >= pool.numel() * pool.element_size() > 20e6
    del pool
    engine.cleanup()
    left = torch.cuda.memory_allocated() - base
    assert left < 0.02 * held, f"{left} of {held} bytes are still held after cleanup"
    with pytest.raises(RuntimeError, match="cleaned up"):
        engine.infer_batch([(prompt, params)])
    other = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="bfloat16"))
    assert other.infer_batch([(prompt, params)])[0].output_ids[0] == before
    other.cleanup()
    engine.initialize()
    with pytest.raises(RuntimeError, match="no weights"):
        engine.infer_batch([(prompt, params)])
    engine.load_state_dict(pw)
    assert engine.infer_batch([(prompt, params)])[0].output_ids[0] == before
    assert engine.model_runner.graph_replays > 0


def test_command_line(models, tmp_path):
    folder, pc, pw = models[("B", "float32")]
    cmd = [sys.executable, "-m", "halite_amd.cli.generate", "--model", folder, "--prompt-ids", "5,17,3,250,9",
           "--prompt-lens", "12", "--prompt-seed", "4", "--stats",
           "sampling.temperature=0", "sampling.max_new_tokens=6", "model.dtype=float32", "server.page_size=16"]
    proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [json.loads(l) for l in proc.stdout.strip().split("\n")]
    assert len(lines) == 2 and lines[0]["input_ids"] == [5, 17, 3, 250, 9]
    for rec in lines:
        want, _, _ = plain_llama.generate(pc, pw, rec["input_ids"], {"temperature": 0.0, "max_new_tokens": 6})
        assert rec["output_ids"] == [want]
    assert "steps" in proc.stderr
    out = tmp_path / "rand"
    cfgfile = tmp_path / "c.json"
    cfgfile.write_text(json.dumps(tiny.TINY_A))
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "halite_make_random_model"), "--config", str(cfgfile),
                           "--out", str(out), "--seed", "3", "--dtype", "float32"], capture_output=True, text=True)
    assert proc.returncode == 0 and (out / "model.safetensors").exists() and (out / "config.json").exists()
    # --random CONFIG.json: the same configuration with weights drawn on the device; the seed decides
    def random_run(seed):
        cmd = [sys.executable, "-m", "halite_amd.cli.generate", "--random", str(cfgfile), "--weights-seed", str(seed),
               "--prompt-ids", "5,17,3", "sampling.temperature=0", "sampling.max_new_tokens=5", "model.dtype=float32"]
        proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        return json.loads(proc.stdout.strip())["output_ids"][0]

    first = random_run(3)
    assert len(first) == 5 and first == random_run(3)
    proc = subprocess.run([sys.executable, "-m", "halite_amd.cli.generate", "--prompt-ids", "1"], cwd=ROOT,
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode != 0 and "--model DIR and --random" in proc.stderr


def test_a_dropped_engine_does_not_disturb_a_capture(models):
    """An engine that is no longer referenced still holds captured graphs until the garbage
    collector finds it; that must not happen while another engine records one."""
    import gc

    folder, pc, pw = models[("A", "float32")]
    server = ServerConfig(kv_cache_num_tokens=512, use_cudagraph=True)
    prompt = tiny.random_tokens(tiny.TINY_A, 12, 3)
    params = {"max_new_tokens": 6, "temperature": 0.0}
    first = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="float32"))
    want = first.infer_batch([(prompt, params)])[0].output_ids[0]
    assert first.model_runner._graphs
    del first  # garbage with reference cycles: only the collector frees it
    old = gc.get_threshold()
    gc.set_threshold(1, 1, 1)  # collect at every opportunity
    try:
        second = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="float32"))
        assert second.infer_batch([(prompt, params)])[0].output_ids[0] == want
    finally:
        gc.set_threshold(*old)


def test_the_engine_serves_on_after_a_refused_or_failed_batch(models):
    """Requests that can never be served are refused before any of the batch is queued,
    and whatever fails later leaves nothing behind: the next batch gives what it gave
    before."""
    folder, pc, pw = models[("A", "float32")]
    cfg = tiny.TINY_A
    engine = InferenceEngine.from_pretrained(folder, ServerConfig(kv_cache_num_tokens=64, page_size=16), ModelConfig(dtype="float32"))
    good = (tiny.random_tokens(cfg, 10, 1), {"max_new_tokens": 5, "temperature": 0.0})
    want = engine.infer_batch([good])[0].output_ids
    refused = [
        ((tiny.random_tokens(cfg, 100, 2), {"max_new_tokens": 20}), "can never fit"),
        ((tiny.random_tokens(cfg, 200, 2), {"max_new_tokens": 2}), "exceeds the context length"),
        (([5, cfg["vocab_size"]], {"max_new_tokens": 2}), "outside the vocabulary"),
        (([], {"max_new_tokens": 2}), "empty prompt"),
        ((tiny.random_tokens(cfg, 5, 2), {"max_new_tokens": 2, "temperature": -1.0}), "temperature"),
        ((tiny.random_tokens(cfg, 5, 2), {"nonsense": 2}), "nonsense"),
    ]
    for bad, message in refused:
        with pytest.raises((ValueError, TypeError), match=message):
            engine.infer_batch([good, bad])  # the good request before it is not left waiting
        assert not engine.scheduler.waiting and not engine.scheduler.running
        assert engine.infer_batch([good])[0].output_ids == want
    # a failure in the middle of the run (the step function raises): the batch is dropped
    calls = {"n": 0}
    step = engine.model_runner.step

    def failing_step(segments, token_feed=None):
        calls["n"] += 1
        if calls["n"] == 3:
            raise RuntimeError("stand-in for a failure inside a step")
        return step(segments, token_feed=token_feed)

    engine.model_runner.step = failing_step
    with pytest.raises(RuntimeError, match="stand-in"):
        engine.infer_batch([good, (tiny.random_tokens(cfg, 7, 3), {"max_new_tokens": 9, "temperature": 0.0})])
    engine.model_runner.step = step
    assert engine.model_runner.cache.idle()
    assert engine.infer_batch([good])[0].output_ids == want


def test_graphs_recorded_ahead_of_time(models):
    """``initialize(capture_graphs=True)`` records the decode graphs of the batch sizes that
    the configuration lists while the engine is idle; generation then replays them and gives
    the tokens of an engine that records at first use."""
    folder, pc, pw = models[("B", "bfloat16")]
    server = ServerConfig(kv_cache_num_tokens=2048, max_seqs_per_forward=6, use_cudagraph=True, cudagraph_step=1)
    prompts = [tiny.random_tokens(tiny.TINY_B, n, 500 + n) for n in (3, 40, 17, 9)]
    batch = [(p, {"max_new_tokens": 10 + 2 * i, "temperature": 0.0}) for i, p in enumerate(prompts)]
    lazy = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="bfloat16"))
    want = [r.output_ids for r in lazy.infer_batch(batch)]
    eager = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="bfloat16"))
    eager.initialize(capture_graphs=True)
    runner = eager.model_runner
    assert sorted(runner._graphs) == [1, 2, 3, 4, 5, 6] and runner.cache.idle()
    replays = runner.graph_replays
    assert [r.output_ids for r in eager.infer_batch(batch)] == want
    assert runner.graph_replays > replays and sorted(runner._graphs) == [1, 2, 3, 4, 5, 6]
    assert runner.capture_graphs([2, 3]) == [1, 2, 3, 4, 5, 6]  # nothing to do
    # the reference's way to list the sizes: multiples of a step, and additional ones; the
    # other sizes get their graphs when a step first has them
    some = InferenceEngine.from_pretrained(
        folder, server.model_copy(update={"cudagraph_step": 4, "cudagraph_additonal_batch_size": (1, 6, 9)}),
        ModelConfig(dtype="bfloat16"))
    some.initialize(capture_graphs=True)
    assert sorted(some.model_runner._graphs) == [1, 4, 6]  # (no more than six requests are live at a time)
    assert [r.output_ids for r in some.infer_batch(batch)] == want
    assert set(some.model_runner._graphs) >= {1, 2, 3, 4, 6}
    # without graphs there is nothing to record
    plain = InferenceEngine.from_pretrained(folder, ServerConfig(kv_cache_num_tokens=512), ModelConfig(dtype="bfloat16"))
    plain.initialize(capture_graphs=True)
    assert plain.model_runner._graphs == {}


def test_stated_model_sizes_are_checked(models):
    """The reference's callers tell its engine the model's sizes (scripts/eval_task.py:148-154);
    here they are read from the model, and what a caller states must agree."""
    folder, pc, pw = models[("B", "bfloat16")]
    cfg = tiny.TINY_B
    server = ServerConfig(kv_cache_num_tokens=256)
    stated = dict(n_heads=cfg["num_attention_heads"], n_key_value_heads=cfg["num_key_value_heads"],
                  head_dim=cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"]),
                  n_layers=cfg["num_hidden_layers"], context_len=128)
    engine = InferenceEngine.from_pretrained(folder, server, ModelConfig(**stated))
    assert len(engine.infer_batch([([3, 4, 5], {"max_new_tokens": 2, "temperature": 0.0})])[0].output_ids[0]) == 2
    with pytest.raises(ValueError, match="n_key_value_heads"):
        InferenceEngine.from_pretrained(folder, server, ModelConfig(**dict(stated, n_key_value_heads=stated["n_key_value_heads"] + 1)))


class LetterTokenizer:
    """Token t is the letter chr(97 + t % 26); no end-of-text token."""

    eos_id = None
    additional_stop_token_ids = None

    def encode(self, text, add_special_tokens=True):
        return [ord(c) - 97 for c in text]

    def decode(self, ids):
        return "".join(chr(97 + t % 26) for t in ids)


@pytest.mark.parametrize("ahead", [0, 1])
def test_stop_strings_through_the_engine(models, ahead):
    """Stop strings need a tokenizer; with one, a request ends with the token that
    completes the string, also when the step after it was launched already."""
    folder, pc, pw = models[("B", "float32")]
    tok = LetterTokenizer()
    server = ServerConfig(kv_cache_num_tokens=2048, use_cudagraph=True, scheduling_steps_ahead=ahead)
    engine = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="float32"), tokenizer=tok)
    prompts = [tiny.random_tokens(tiny.TINY_B, n, 600 + n) for n in (5, 12, 30)]
    free = engine.infer_batch([(p, {"max_new_tokens": 30, "temperature": 0.0}) for p in prompts])
    texts = [tok.decode(r.output_ids[0]) for r in free]
    stops = [t[10:13] for t in texts]
    got = engine.infer_batch([(p, {"max_new_tokens": 30, "temperature": 0.0, "stop": s}) for p, s in zip(prompts, stops)])
    for r, full, text, s in zip(got, free, texts, stops):
        cut = text.index(s) + len(s)
        assert r.output_ids[0] == full.output_ids[0][:cut] and r.finish_reason == ["stop"]
    assert engine.model_runner.cache.idle()
    with pytest.raises(ValueError, match="tokenizer"):
        InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype="float32")).infer_batch(
            [(prompts[0], {"max_new_tokens": 3, "stop": "ab"})])


def test_the_bench_line_keeps_its_contract():
    """One JSON line with the keys that whoever runs ``bench.py`` reads (here with one layer,
    a short context and a short prompt, so that it takes seconds); more than one GPU is
    refused in one line with exit status 2."""
    cmd = [sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "1", "--steps", "4", "--warmup", "2",
           "--context", "1024", "--prefill-tokens", "256", "--no-extras"]
    proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().split("\n")
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 4 and rec["warmup"] == 2 and rec["higher_is_better"] is True
    assert rec["dtype"] == "bf16" and rec["unit"] == "tok/s" and rec["value"] > 0
    assert abs(rec["value"] - 8 / rec["ms_per_step"] * 1e3) < 0.01 * rec["value"]
    config = rec["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["layers"] == 1 and config["layers_of_model"] == 32 and config["global_batch"] == 8 and config["seq_len"] == 1024
    for key in ("hidden_size", "heads", "kv_heads", "head_dim", "intermediate_size", "vocab_size"):
        assert config[key] > 0
    assert set(rec["prefill"]) >= {"value", "tokens", "ms", "frac"} and rec["prefill"]["tokens"] == 256
    roof = rec["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert rec["points"]["decode_b1"] > 0 and rec["points"]["decode_b64"] > 0
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], cwd=ROOT, capture_output=True,
                          text=True, timeout=120)
    assert proc.returncode == 2 and len((proc.stdout + proc.stderr).strip().split("\n")) == 1
