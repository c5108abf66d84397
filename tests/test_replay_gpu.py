"""Replay on the GPU: the same requests whole, with the last 32 tokens decoded one by
one, in portions of changing size, and mixed with other requests so that pages are used
again; in 32-bit and in bfloat16; each compared with the plain implementation run on
the whole sequence.  A difference that shows in one way of cutting only is a fault of
the cache or the batch."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama
import replay
import tiny
from halite_amd.config import ModelConfig, ServerConfig
from halite_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 5e-5, "bfloat16": 2.5e-2}  # of the largest logit
CONFIGS = {"A": tiny.TINY_A, "B": tiny.TINY_B, "C": tiny.TINY_C}
LENGTHS = {"A": [5, 17, 33, 64, 100, 128], "B": [1, 40, 100, 2, 256, 65], "C": [130, 64, 31, 200, 3, 97]}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """One model folder per configuration and stored type, and the plain logits of
    every request's whole sequence (from the stored, i.e. rounded, weights)."""
    out = {}
    for name, cfg in CONFIGS.items():
        weights = tiny.random_weights(cfg, seed=11 + len(name), std=0.06)
        requests = {f"r{i}": tiny.random_tokens(cfg, n, 100 + i) for i, n in enumerate(LENGTHS[name])}
        for dtype, store in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
            folder = str(tmp_path_factory.mktemp(f"{name}_{dtype}"))
            tiny.write_model_folder(folder, cfg, weights, store)
            pc, pw = plain_llama.read_model_folder(folder)
            ref = {rid: plain_llama.forward(pc, pw, toks) for rid, toks in requests.items()}
            out[(name, dtype)] = (folder, requests, ref)
    return out


def make_runner(folder, dtype, tokens, page_size=64, **server_options):
    server = ServerConfig(kv_cache_num_tokens=tokens, page_size=page_size, max_seqs_per_forward=8, **server_options)
    return ModelRunner.from_pretrained(folder, server, ModelConfig(dtype=dtype))


SCHEDULES = {
    "whole": replay.whole,
    "tail": replay.tail_one_by_one,
    "portions": replay.portions,
    "mixed": replay.mixed,
}


# B has heads of 32: with pages of 32 or 64 tokens its bf16 cache lies in the matrix-core
# kernel's own order, with pages of 16 row by row
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("name,page", [("A", 64), ("B", 16), ("B", 32), ("B", 64), ("C", 64)])
def test_schedules(folders, name, page, schedule, dtype):
    folder, requests, ref = folders[(name, dtype)]
    trace = SCHEDULES[schedule](requests)
    # exactly as many pages as the trace needs at its peak: they are used again
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, page), page)
    tiled = [runner.cache.layer_pages(r.index).tiled for r in runner.model.runs]
    assert all(t == (dtype == "bfloat16" and name == "B" and page >= 32) for t in tiled)
    # whatever free or not yet written slots hold must never reach a result
    for g in runner.cache.groups:
        g.storage.fill_(float("nan"))
    logits = replay.run_trace(runner, trace)
    rows = replay.collect(trace, logits, CONFIGS[name]["vocab_size"])
    assert sum(len(v) for v in rows.values()) > 0
    replay.compare(rows, ref, TOL[dtype])
    assert runner.cache.idle()


@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("name,page", [("B", 16), ("B", 64), ("C", 64)])
def test_schedules_on_row_major_weights(folders, name, page, schedule, monkeypatch):
    """bfloat16 without the second, tiled copy of the matrices (a model too large for it, or
    ``decode_weight_copy="off"``): steps of few tokens then take the norm, the products on
    the row-major matrices and the rotation as kernels of their own, none of the fused ones."""
    from halite_amd.kernels import ops

    fused = []
    for fn in ("qkv_rope_append", "gemm_bf16_skinny_norm"):
        monkeypatch.setattr(ops, fn, lambda *a, _n=fn, **kw: fused.append(_n))
    folder, requests, ref = folders[(name, "bfloat16")]
    trace = SCHEDULES[schedule](requests)
    runner = make_runner(folder, "bfloat16", replay.peak_tokens(trace, page), page, decode_weight_copy="off")
    assert not runner.model.build.tiled_weights
    for g in runner.cache.groups:
        g.storage.fill_(float("nan"))
    rows = replay.collect(trace, replay.run_trace(runner, trace), CONFIGS[name]["vocab_size"])
    replay.compare(rows, ref, TOL["bfloat16"])
    assert runner.cache.idle() and not fused


def test_bfloat16_run_of_a_folder_stored_in_float32(folders):
    """Tensors stored in 32-bit stay so: the products then run on the float32 kernels
    with bfloat16 activations, cache and attention."""
    folder, requests, ref = folders[("B", "float32")]
    trace = replay.mixed(requests, seed=2)
    runner = make_runner(folder, "bfloat16", replay.peak_tokens(trace))
    assert runner.model.embedding.weight.dtype == torch.float32
    assert runner.cache.groups[0].storage.dtype == torch.bfloat16
    rows = replay.collect(trace, replay.run_trace(runner, trace), 512)
    replay.compare(rows, ref, TOL["bfloat16"])


def test_a_reader_that_does_not_scale_gets_whole_rows(folders, monkeypatch):
    """Where the product before a norm has prepared its rows but the part after cannot
    finish the norm in its own product (a gated feed-forward too large at 17 to 32 rows:
    forced here by the threshold), the rows are made whole by a kernel of their own, and
    the logits are those of the plain implementation."""
    from halite_amd.kernels import ops

    made = []
    whole = ops.NormedRows.materialize
    monkeypatch.setattr(ops.NormedRows, "materialize", lambda self: made.append(self.shape[0]) or whole(self))
    monkeypatch.setattr(ops, "GATED_MID_ELEMENTS", 0)
    folder, requests, ref = folders[("B", "bfloat16")]
    trace = replay.portions({"r2": requests["r2"], "r4": requests["r4"]}, sizes=(20, 31, 17, 24, 32, 19))
    runner = make_runner(folder, "bfloat16", replay.peak_tokens(trace))
    rows = replay.collect(trace, replay.run_trace(runner, trace), 512)
    replay.compare(rows, ref, TOL["bfloat16"])
    assert made and all(17 <= m <= 32 for m in made)


def test_steps_of_few_tokens_take_the_fused_kernels(folders, monkeypatch):
    """With the tiled weight copy a bf16 step of at most 32 tokens runs rotation and append
    inside the q, k, v product and every norm but the first and the last inside the
    products around it; a larger step and the 32-bit path use the kernels of their own.
    (Their results are compared with the plain implementation by the schedules above.)"""
    from halite_amd.engine.batch import Segment
    from halite_amd.kernels import ops

    calls = {}
    for name in ("rmsnorm", "rope_append", "qkv_rope_append", "gemm_bf16_skinny_norm"):
        def counted(*a, _f=getattr(ops, name), _n=name, **kw):
            calls[_n] = calls.get(_n, 0) + 1
            return _f(*a, **kw)
        monkeypatch.setattr(ops, name, counted)
    folder, requests, _ = folders[("B", "bfloat16")]
    layers = tiny.TINY_B["num_hidden_layers"]
    toks = requests["r2"]
    runner = make_runner(folder, "bfloat16", 128)
    slot = runner.admit()
    runner.step([Segment(slot, 0, toks[:40], [39])])
    assert calls == {"rmsnorm": 2 * layers + 1, "rope_append": layers}
    # per layer: o-proj (prepares the next norm), gate/up (scaled), down (prepares) = 3,
    # less the last down-projection, whose norm is the model's final one over wanted rows
    fused = {"rmsnorm": 2, "qkv_rope_append": layers, "gemm_bf16_skinny_norm": 3 * layers - 1}
    calls.clear()
    runner.step([Segment(slot, 40, toks[40:60], [19])])  # 17 to 32 tokens: two row tiles per wave
    # ... where that is the faster way: not for the down-projection, whose rows are long, so
    # the norm after it is a kernel
    assert calls == {"rmsnorm": 2 + layers - 1, "qkv_rope_append": layers, "gemm_bf16_skinny_norm": 2 * layers}
    calls.clear()
    runner.step([Segment(slot, 60, toks[60:63], [2])])
    assert calls == fused
    runner.free(slot)
    calls.clear()
    folder32, _, _ = folders[("B", "float32")]
    runner = make_runner(folder32, "float32", 128)
    slot = runner.admit()
    runner.step([Segment(slot, 0, toks[:3], [2])])
    assert calls == {"rmsnorm": 2 * layers + 1, "rope_append": layers}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_agree_with_each_other(folders, dtype):
    """The logits at a position do not depend on how the tokens were cut, beyond
    rounding: far tighter than the distance to the plain implementation in bf16."""
    folder, requests, _ = folders[("C", dtype)]
    results = []
    for schedule in ("whole", "tail", "portions"):
        trace = SCHEDULES[schedule](requests)
        runner = make_runner(folder, dtype, replay.peak_tokens(trace))
        results.append(replay.collect(trace, replay.run_trace(runner, trace), 331))
    tol = 2e-5 if dtype == "float32" else 1.5e-2
    for other in results[1:]:
        for rid in results[0]:
            a = torch.stack([results[0][rid][p] for p in sorted(results[0][rid])])
            b = torch.stack([other[rid][p] for p in sorted(other[rid])])
            assert float((a - b).abs().max()) <= tol * max(1.0, float(a.abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_pages_and_other_page_sizes(folders, dtype):
    folder, requests, ref = folders[("A", dtype)]
    trace = replay.mixed(requests, seed=3)
    # (bfloat16 pages of 1 and 4 tokens: the plain attention kernel on a bfloat16 cache)
    for page in ([1, 4, 8, 16] if dtype == "float32" else [1, 4, 8, 16, 32]):
        runner = make_runner(folder, dtype, replay.peak_tokens(trace, page), page)
        for g in runner.cache.groups:
            g.storage.fill_(float("nan"))
        rows = replay.collect(trace, replay.run_trace(runner, trace), 256)
        replay.compare(rows, ref, TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(folders, dtype):
    folder, requests, ref = folders[("C", dtype)]
    rid = "r3"  # 200 tokens
    toks = requests[rid]
    # every token on its own, from an empty cache
    trace = [{"step": i, "entries": [{"id": rid, "tokens": [t], "want": [0]}], "end": [rid] if i == len(toks) - 1 else []}
             for i, t in enumerate(toks)]
    runner = make_runner(folder, dtype, 256)
    rows = replay.collect(trace, replay.run_trace(runner, trace), 331)
    replay.compare(rows, ref, TOL[dtype])
    # the first tokens of a sequence: one token, two tokens
    for n in (1, 2):
        trace = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:n], "want": list(range(n))}], "end": [rid]}]
        rows = replay.collect(trace, replay.run_trace(runner, trace), 331)
        replay.compare(rows, ref, TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(folders, dtype, tmp_path):
    """The program itself, as a user runs it: JSON lines in, <step>.f32 files out."""
    folder, requests, ref = folders[("B", dtype)]
    trace = replay.mixed(requests, seed=1)
    out = tmp_path / "out"
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", str(out), "--max-tokens", str(replay.peak_tokens(trace))]
    proc = subprocess.run(cmd, input="\n".join(json.dumps(s) for s in trace) + "\n", text=True,
                          capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l] == [f"done {s['step']}" for s in trace]
    logits = {}
    for s in trace:
        n_want = sum(len(e["want"]) for e in s["entries"])
        path = out / f"{s['step']}.f32"
        if n_want == 0:
            assert not path.exists()
            continue
        logits[s["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n_want, 512))
    rows = replay.collect(trace, logits, 512)
    replay.compare(rows, ref, TOL[dtype])


def test_trace_run_step_by_step(folders, tmp_path):
    """A step is sent only after the line ``done <step>`` of the one before has come back;
    by then the step's file is complete."""
    folder, requests, ref = folders[("A", "float32")]
    trace = replay.portions({k: requests[k] for k in list(requests)[:3]})
    out = tmp_path / "out"
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
           "--out", str(out), "--max-tokens", str(replay.peak_tokens(trace))]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)
    logits = {}
    try:
        for s in trace:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {s['step']}"
            n_want = sum(len(e["want"]) for e in s["entries"])
            if n_want:
                data = np.fromfile(out / f"{s['step']}.f32", dtype="<f4")
                assert data.size == n_want * 256
                logits[s["step"]] = torch.from_numpy(data.reshape(n_want, 256))
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    replay.compare(replay.collect(trace, logits, 256), ref, TOL["float32"])


def test_refusals(folders):
    from halite_amd.cache import NoSpace
    from halite_amd.engine.batch import Segment
    from halite_amd.engine.runner import StepError

    folder, requests, _ = folders[("A", "float32")]
    runner = make_runner(folder, "float32", 128)
    s = runner.admit()
    with pytest.raises(StepError, match="outside the vocabulary"):
        runner.step([Segment(s, 0, [5, 256], [0])])
    with pytest.raises(StepError, match="are cached"):
        runner.step([Segment(s, 3, [5], [0])])
    with pytest.raises(StepError, match="twice"):
        runner.step([Segment(s, 0, [5], [0]), Segment(s, 1, [6], [0])])
    with pytest.raises(StepError, match="context length"):
        runner.step([Segment(s, 0, list(range(129)), [])])
    runner.step([Segment(s, 0, list(range(100)), [])])
    s2 = runner.admit()
    with pytest.raises(NoSpace):
        runner.step([Segment(s2, 0, list(range(100)), [])])  # 2 pages of 64 in all
    assert runner.cache.length(s2) == 0
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_through_a_captured_graph(folders, dtype):
    """Decode-only steps replayed from a HIP graph: every replay is checked, with
    eager work (a prompt of another request, a change of the batch size) between
    replays, against the plain implementation and against the eager engine."""
    folder, requests, ref = folders[("C", dtype)]
    server = ServerConfig(kv_cache_num_tokens=1024, page_size=16, max_seqs_per_forward=8, use_cudagraph=True)
    runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype=dtype))
    a, b, c = requests["r0"], requests["r3"], requests["r1"]  # 130, 200, 64 tokens
    trace = [{"step": 0, "entries": [{"id": "a", "tokens": a[:60], "want": [59]}, {"id": "b", "tokens": b[:100], "want": []}], "end": []}]
    pa, pb = 60, 100
    for i in range(60):
        entries = [{"id": "a", "tokens": [a[pa]], "want": [0]}, {"id": "b", "tokens": [b[pb]], "want": [0]}]
        pa, pb = pa + 1, pb + 1
        trace.append({"step": len(trace), "entries": entries, "end": []})
        if i == 20:  # an eager prompt between two replays
            trace.append({"step": len(trace), "entries": [{"id": "c", "tokens": c, "want": [63]}], "end": ["c"]})
    trace[-1]["end"] = ["a"]
    for i in range(30):  # the batch shrinks to one request: another graph
        trace.append({"step": len(trace), "entries": [{"id": "b", "tokens": [b[pb]], "want": [0]}], "end": []})
        pb += 1
    trace[-1]["end"] = ["b"]
    logits = replay.run_trace(runner, trace)
    assert runner.graph_replays >= 80 and sorted(runner._graphs) == [1, 2]
    # most replays ran a step that the host had put together while the GPU worked on the one
    # before; the prompt in between, the request that ended and the first steps did not
    assert 70 <= runner.steps_taken_ahead < runner.graph_replays
    rows = replay.collect(trace, logits, 331)
    ref2 = {"a": ref["r0"], "b": ref["r3"], "c": ref["r1"]}
    replay.compare(rows, ref2, TOL[dtype])
    eager = make_runner(folder, dtype, 1024, 16)
    rows_eager = replay.collect(trace, replay.run_trace(eager, trace), 331)
    for rid in rows:
        for p in rows[rid]:
            d = float((rows[rid][p] - rows_eager[rid][p]).abs().max())
            assert d <= (1e-6 if dtype == "float32" else 2e-2), (rid, p, d)


ODD = {
    # a head size that is no multiple of 16 and a width that is no multiple of 8: the plain
    # attention kernel and the library product serve the bfloat16 path
    "head20": dict(tiny.TINY_A, hidden_size=60, num_attention_heads=3, num_key_value_heads=1, head_dim=20,
                   intermediate_size=70, vocab_size=101),
    "head24": dict(tiny.TINY_A, hidden_size=72, num_attention_heads=3, num_key_value_heads=3, head_dim=24,
                   intermediate_size=100, vocab_size=257),
    # heads of 96 and 256: tiled pages; 256 is the largest head and takes steps of 32 keys
    "head96": dict(tiny.TINY_A, hidden_size=192, num_attention_heads=2, num_key_value_heads=1, head_dim=96,
                   intermediate_size=520, vocab_size=1000, max_position_embeddings=512),
    "head256": dict(tiny.TINY_A, hidden_size=256, num_attention_heads=2, num_key_value_heads=2, head_dim=256,
                    intermediate_size=384, vocab_size=333, max_position_embeddings=512, tie_word_embeddings=True),
    # no head_dim in the file: hidden_size / heads
    "derived": {k: v for k, v in dict(tiny.TINY_A, hidden_size=96, num_attention_heads=6, num_key_value_heads=2,
                                      intermediate_size=128).items() if k != "head_dim"},
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ODD))
def test_other_sizes(name, dtype, tmp_path):
    cfg = ODD[name]
    weights = tiny.random_weights(cfg, seed=3, std=0.06)
    longest = 128 if cfg["max_position_embeddings"] < 200 else 300
    requests = {f"r{i}": tiny.random_tokens(cfg, n, 50 + i) for i, n in enumerate([70, 9, longest, 33])}
    folder = str(tmp_path / "model")
    tiny.write_model_folder(folder, cfg, weights, torch.float32 if dtype == "float32" else torch.bfloat16)
    pc, pw = plain_llama.read_model_folder(folder)
    ref = {rid: plain_llama.forward(pc, pw, toks) for rid, toks in requests.items()}
    for make in (replay.tail_one_by_one, replay.portions, replay.mixed):
        trace = make(requests)
        runner = make_runner(folder, dtype, replay.peak_tokens(trace))
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab_size"])
        replay.compare(rows, ref, TOL[dtype])


LLAMA_8B_LAYERS = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256, num_hidden_layers=2,
    rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False,
    hidden_act="silu", attention_bias=False, mlp_bias=False,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)


@pytest.mark.parametrize("dtype,weight_copy", [("float32", "auto"), ("bfloat16", "auto"), ("bfloat16", "off")])
def test_layers_of_the_8b_shape(dtype, weight_copy, tmp_path):
    """Two layers with every size of Llama-3.1-8B (width 4096, 32 heads over 8 groups of
    128, feed-forward 14336, vocabulary 128256, llama3 frequency scaling), weights
    N(0, 0.02): the kernels at the sizes that the benchmark runs; in bfloat16 with and
    without the tiled copy of the matrices (without: the way of the 70B shape)."""
    cfg = LLAMA_8B_LAYERS
    weights = tiny.random_weights(cfg, seed=11, std=0.02)
    requests = {f"r{i}": tiny.random_tokens(cfg, n, 70 + i) for i, n in enumerate([70, 9, 200, 33])}
    folder = str(tmp_path / "model")
    tiny.write_model_folder(folder, cfg, weights, torch.float32 if dtype == "float32" else torch.bfloat16)
    del weights
    pc, pw = plain_llama.read_model_folder(folder)
    ref = {rid: plain_llama.forward(pc, pw, toks) for rid, toks in requests.items()}
    del pw
    runner = None
    for make in (replay.whole, replay.tail_one_by_one, replay.portions, replay.mixed):
        trace = make(requests)
        del runner
        runner = make_runner(folder, dtype, replay.peak_tokens(trace), decode_weight_copy=weight_copy)
        assert runner.model.build.tiled_weights == (dtype == "bfloat16" and weight_copy == "auto")
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab_size"])
        replay.compare(rows, ref, TOL[dtype])


def test_eight_layers_of_the_8b_shape_within_the_bounds_of_the_number_format():
    """At depth the bfloat16 engine's distance from float32 arithmetic is measured against
    that of the plain implementation rounding to bfloat16 at the same places, under all
    four schedules; float32 against 1e-4.  ``tests/full_depth_equality.py`` states the
    bounds and runs the same with all 32 layers."""
    import full_depth_equality

    lines, missed = full_depth_equality.run(8, [70, 9, 150, 33])
    assert not missed, "\n".join(missed + lines)


def test_the_pool_is_sized_from_free_memory(folders, monkeypatch):
    """Without ``kv_cache_num_tokens`` the pool takes what the reference's formula gives
    (src/halite/transformers/infer/engine/model_runner.py:117-131: free memory less the
    share of the whole that ``memory_fraction_static`` keeps back, over the bytes of a
    cached token), capped at what ``max_seqs_per_forward`` requests of the context length
    could hold; and the engine generates with it."""
    from halite_amd.engine.engine import InferenceEngine

    folder, requests, ref = folders[("B", "bfloat16")]
    cfg = tiny.TINY_B
    per_token = 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * cfg["num_hidden_layers"] * 2  # keys and values, bf16
    GiB = 1 << 30
    total, fraction, page = 4 * GiB, 0.88, 16
    free = int(total * (1 - fraction)) + 300_000  # what the formula leaves: 300,000 bytes
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (free, total))
    server = ServerConfig(kv_cache_num_tokens=None, page_size=page, max_seqs_per_forward=64)
    runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype="bfloat16", memory_fraction_static=fraction))
    usable = free - total * (1 - fraction)
    reference_tokens = int(usable // per_token)
    assert runner.cache.num_pages == int(usable // (per_token * page)) and runner.cache.num_pages > 40
    # (a page number is reserved, and the pool holds whole pages)
    assert reference_tokens - 2 * page < runner.cache.token_capacity <= reference_tokens
    assert runner.cache.token_capacity == runner.max_total_tokens == (runner.cache.num_pages - 1) * page
    engine = InferenceEngine(runner)
    toks = requests["r1"]
    out = engine.infer_batch([(0, toks[:30], {"max_new_tokens": 4, "temperature": 0.0})])[0].output_ids[0]
    assert len(out) == 4
    logits = plain_llama.forward(*plain_llama.read_model_folder(folder), toks[:30] + out)
    for j, tok in enumerate(out):  # the plain implementation's best token, or within rounding of it
        row = logits[29 + j]
        assert float(row.max() - row[tok]) <= TOL["bfloat16"] * max(1.0, float(row.abs().max()))
    # plenty of memory: the cap
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (3 * GiB, total))
    capped = ModelRunner.from_pretrained(folder, ServerConfig(kv_cache_num_tokens=None, page_size=page, max_seqs_per_forward=8),
                                         ModelConfig(dtype="bfloat16", memory_fraction_static=fraction))
    assert capped.cache.num_pages == 8 * (cfg["max_position_embeddings"] // page) + 1
    # none: an error that says so
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (int(total * (1 - fraction)), total))
    with pytest.raises(RuntimeError, match="no device memory is left"):
        ModelRunner.from_pretrained(folder, server, ModelConfig(dtype="bfloat16", memory_fraction_static=fraction))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_with_the_heads_of_the_8b_shape(dtype, tmp_path):
    """Prompts of thousands of tokens through two layers with 32 heads over 8 groups of
    128 (a small vocabulary keeps the test short): the prompt kernels walk dozens of
    blocks of keys, whole, in portions and mixed with other requests."""
    cfg = dict(LLAMA_8B_LAYERS, vocab_size=4096)
    weights = tiny.random_weights(cfg, seed=11, std=0.02)
    requests = {f"r{i}": tiny.random_tokens(cfg, n, 70 + i) for i, n in enumerate([3000, 700, 33])}
    folder = str(tmp_path / "model")
    tiny.write_model_folder(folder, cfg, weights, torch.float32 if dtype == "float32" else torch.bfloat16)
    del weights
    pc, pw = plain_llama.read_model_folder(folder)
    ref = {rid: plain_llama.forward(pc, pw, toks) for rid, toks in requests.items()}
    del pw
    for make in (replay.whole, replay.portions, replay.mixed):
        trace = make(requests)
        runner = make_runner(folder, dtype, replay.peak_tokens(trace))
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab_size"])
        replay.compare(rows, ref, TOL[dtype])
        del runner


def drawn_configuration(rng) -> dict:
    """A Llama 3 configuration with every size and option drawn: head sizes that the bf16
    matrix-core attention serves and others, groups of one to eight heads, widths and
    vocabularies that are no powers of two, some of them no multiples of eight."""
    kv = rng.choice([1, 1, 2, 3, 4])
    heads = kv * rng.choice([1, 2, 3, 4, 5, 8])
    cfg = {
        "architectures": ["LlamaForCausalLM"], "vocab_size": rng.randint(50, 3000), "hidden_size": rng.choice([8, 8, 2]) * rng.randint(2, 40),
        "num_hidden_layers": rng.randint(1, 3), "num_attention_heads": heads, "num_key_value_heads": kv,
        "head_dim": rng.choice([16, 32, 48, 64, 80, 96, 112, 128] if rng.random() < 0.7 else [8, 24, 40, 56, 72, 160, 256]),
        "intermediate_size": rng.choice([8, 8, 2]) * rng.randint(3, 90), "rms_norm_eps": rng.choice([1e-5, 1e-6, 3e-4]),
        "rope_theta": rng.choice([10000.0, 500000.0, 77777.0]), "max_position_embeddings": rng.choice([96, 300, 700]),
        "tie_word_embeddings": rng.random() < 0.5,
    }
    if rng.random() < 0.5:
        cfg["rope_scaling"] = {"rope_type": "llama3", "factor": rng.choice([2.0, 8.0, 32.0]), "low_freq_factor": 1.0,
                               "high_freq_factor": rng.choice([2.0, 4.0]), "original_max_position_embeddings": rng.choice([32, 64, 128])}
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations_under_the_mixed_schedule(dtype, seed, tmp_path):
    """Configurations, page sizes, request lengths and the trace drawn from a seed: up to four
    live requests, portions beside decoded tokens, a pool of exactly the trace's peak filled
    with NaN, with and without graphs.  float32 within the suite's tolerance.  bfloat16 is
    measured with the yardstick of the check at depth, since the format's cost depends on the
    configuration: the plain implementation rounding to bfloat16 at the same places; the
    engine's root mean square distance from float32 arithmetic may be 1.3 times that one's,
    its largest difference twice that one's (the largest of many scatters)."""
    import random

    import full_depth_equality as depth

    rng = random.Random(1000 * seed + (dtype == "bfloat16"))
    cfg = drawn_configuration(rng)
    page = rng.choice([8, 16, 32, 64, 128] if dtype == "bfloat16" else [1, 4, 8, 16, 32, 64])
    lengths = [rng.randint(1, cfg["max_position_embeddings"]) for _ in range(rng.randint(2, 6))]
    weights = tiny.random_weights(cfg, seed=rng.randint(0, 999), std=0.06)
    requests = {f"r{i}": tiny.random_tokens(cfg, n, rng.randint(0, 9999)) for i, n in enumerate(lengths)}
    folder = str(tmp_path / "model")
    tiny.write_model_folder(folder, cfg, weights, torch.float32 if dtype == "float32" else torch.bfloat16)
    pc, pw = plain_llama.read_model_folder(folder)  # (the stored, i.e. rounded, weights)
    ref = {rid: plain_llama.forward(pc, pw, toks) for rid, toks in requests.items()}
    trace = replay.mixed(requests, seed=rng.randint(0, 999))
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, page), page_size=page, use_cudagraph=rng.random() < 0.5)
    for g in runner.cache.groups:
        g.storage.fill_(float("nan"))
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab_size"])
    assert runner.cache.idle()
    what = f"{cfg}, pages of {page}, requests of {lengths}"
    worst, rms, _ = depth.distance(rows, ref)
    if dtype == "float32":
        assert worst <= TOL["float32"], what
        return
    rounding = {rid: plain_llama.forward(pc, pw, toks, round_to=torch.bfloat16) for rid, toks in requests.items()}
    e_worst, e_rms, _ = depth.distance({rid: {p: rounding[rid][p] for p in rows[rid]} for rid in rows}, ref)
    assert rms <= 1.3 * e_rms and worst <= 2.0 * e_worst, f"{what}: largest {worst:.3e} (format {e_worst:.3e}), rms {rms:.3e} (format {e_rms:.3e})"


@pytest.mark.parametrize("page_size", [1, 4])
def test_pages_taken_for_a_step_ahead_come_back_when_another_step_needs_them(folders, page_size):
    """With graphs a decode step's successor is put together while the GPU works, pages and
    all.  If another step comes instead, one that needs the pool's last pages for another
    request, the pages taken ahead are given back: a pool of exactly the trace's peak
    serves the trace."""
    folder, requests, ref = folders[("A", "float32")]
    a, b = requests["r1"], requests["r2"]
    assert len(a) >= 12 and len(b) >= 9
    trace = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [8]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": [0]}], "end": []},  # recorded
        {"step": 2, "entries": [{"id": "a", "tokens": a[10:11], "want": [0]}], "end": []},  # replayed
        # replayed; its successor is prepared, with a page for a's thirteenth token (a's 12 fill three pages of 4)
        {"step": 3, "entries": [{"id": "a", "tokens": a[11:12], "want": [0]}], "end": []},
        {"step": 4, "entries": [{"id": "b", "tokens": b[:8], "want": [7]}], "end": ["a"]},  # the peak: a's 12 and b's 8
        {"step": 5, "entries": [{"id": "b", "tokens": b[8:9], "want": [0]}], "end": ["b"]},
    ]
    peak = replay.peak_tokens(trace, page_size)
    assert peak == 20
    runner = make_runner(folder, "float32", peak, page_size=page_size, use_cudagraph=True)
    for g in runner.cache.groups:
        g.storage.fill_(float("nan"))
    given_back = []
    release = runner._release_pages_taken_ahead
    runner._release_pages_taken_ahead = lambda: given_back.append(release()) or given_back[-1]
    rows = replay.collect(trace, replay.run_trace(runner, trace), CONFIGS["A"]["vocab_size"])
    replay.compare(rows, {"a": ref["r1"], "b": ref["r2"]}, TOL["float32"])
    assert given_back == [True]  # (the case is the one that is meant)
    assert runner.graph_replays >= 1 and runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_decode_graph_serves_key_ranges_of_one_piece_and_of_several(dtype, tmp_path):
    """A decode step's attention leaves a short key range whole (one workgroup, no partial
    results) and cuts a longer one into pieces that the merge kernel joins.  One recorded step
    serves both: a request decodes across the length where the second piece begins, beside one
    that stays below it."""
    from halite_amd.kernels import attention as attention_kernels

    cfg = dict(LLAMA_8B_LAYERS, vocab_size=4096)
    weights = tiny.random_weights(cfg, seed=12, std=0.02)
    a, b = tiny.random_tokens(cfg, 1060, 80), tiny.random_tokens(cfg, 90, 81)
    folder = str(tmp_path / "model")
    tiny.write_model_folder(folder, cfg, weights, torch.float32 if dtype == "float32" else torch.bfloat16)
    del weights
    pc, pw = plain_llama.read_model_folder(folder)
    ref = {"a": plain_llama.forward(pc, pw, a), "b": plain_llama.forward(pc, pw, b)}
    del pw
    edge = 2 * attention_kernels.MIN_PIECE_KEYS
    assert edge + 30 <= len(a)
    trace = [{"step": 0, "entries": [{"id": "a", "tokens": a[: edge - 30], "want": []}, {"id": "b", "tokens": b[:30], "want": []}], "end": []}]
    for i in range(60):  # a's context passes the edge at i = 30
        trace.append({"step": len(trace), "entries": [{"id": "a", "tokens": [a[edge - 30 + i]], "want": [0]},
                                                       {"id": "b", "tokens": [b[30 + i]], "want": [0]}], "end": []})
    trace[-1]["end"] = ["a", "b"]
    server = ServerConfig(kv_cache_num_tokens=1280, page_size=64, max_seqs_per_forward=4, use_cudagraph=True)
    runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype=dtype))
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab_size"])
    assert sorted(runner._graphs) == [2] and runner.graph_replays >= 56
    replay.compare(rows, ref, TOL[dtype])


def test_twenty_heads_to_a_key_value_head_decode_from_a_graph(tmp_path):
    """More than 16 heads share a key/value head: a token's rows are two tiles, and a decode
    step still has one-tile items only, so it is recorded and replayed like any other; its
    key ranges are cut into pieces (40 tiles and key/value heads: six a tile at most) that
    the attention kernel merges itself."""
    cfg = dict(tiny.TINY_A, hidden_size=320, num_attention_heads=20, num_key_value_heads=1, head_dim=16,
               intermediate_size=96, num_hidden_layers=2, vocab_size=331, max_position_embeddings=2048)
    weights = tiny.random_weights(cfg, seed=5, std=0.06)
    a, b = tiny.random_tokens(cfg, 1300, 90), tiny.random_tokens(cfg, 60, 91)
    folder = str(tmp_path / "model")
    tiny.write_model_folder(folder, cfg, weights, torch.bfloat16)
    pc, pw = plain_llama.read_model_folder(folder)
    ref = {"a": plain_llama.forward(pc, pw, a), "b": plain_llama.forward(pc, pw, b)}
    trace = [{"step": 0, "entries": [{"id": "a", "tokens": a[:1250], "want": []}, {"id": "b", "tokens": b[:20], "want": []}], "end": []}]
    for i in range(40):
        trace.append({"step": len(trace), "entries": [{"id": "a", "tokens": [a[1250 + i]], "want": [0]},
                                                       {"id": "b", "tokens": [b[20 + i]], "want": [0]}], "end": []})
    trace[-1]["end"] = ["a", "b"]
    server = ServerConfig(kv_cache_num_tokens=1536, page_size=64, max_seqs_per_forward=4, use_cudagraph=True)
    runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype="bfloat16"))
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab_size"])
    assert sorted(runner._graphs) == [2] and runner.graph_replays >= 36
    replay.compare(rows, ref, TOL["bfloat16"])
