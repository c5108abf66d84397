"""Benchmark: decode tokens a second and prefill tokens a second at the Llama-3.1-8B
shape with seeded random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The default run decodes a batch of 8 requests whose contexts end at the configured
context length (8,192 tokens); a step is one decode step of the engine: building the
batch, the forward pass from the paged cache, greedy sampling and reading the tokens
back.  The same line carries the prefill of one 2,048-token prompt, the decode step's
fraction of the HBM roofline, decode rates at batch 1 and 64 (contexts that end at 8,192
and 512-token prompts), the host's share of a step, what the kernel families of a step
reach against their rooflines (HIP events around each call of an eager step), and what
this GPU gives a plain copy and a large library product (the attainable figures beside
the published peaks).  ``--more-points`` adds further batches, contexts and prompt lengths.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

LLAMA_3_1_8B = dict(
    architectures=["LlamaForCausalLM"],
    vocab_size=128256,
    hidden_size=4096,
    num_hidden_layers=32,
    num_attention_heads=32,
    num_key_value_heads=8,
    head_dim=128,
    intermediate_size=14336,
    rms_norm_eps=1e-5,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=131072,
    tie_word_embeddings=False,
)


LLAMA_3_2_3B = dict(
    LLAMA_3_1_8B,
    hidden_size=3072,
    num_hidden_layers=28,
    num_attention_heads=24,
    intermediate_size=8192,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=True,
)

LLAMA_3_1_70B = dict(
    LLAMA_3_1_8B,
    hidden_size=8192,
    num_hidden_layers=80,
    num_attention_heads=64,
    intermediate_size=28672,
)


def layer_params(c) -> int:
    d, f = c.hidden_size, c.intermediate_size
    qkv = (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim * d
    return qkv + c.num_attention_heads * c.head_dim * d + 3 * f * d + 2 * d


def decode_bytes(c, n_layers, batch, kv_tokens, elt=2) -> float:
    """What a decode step has to read: every weight it uses once (layers, final
    norm, head; of the embedding only the batch's rows) and the cached keys and
    values of the live requests."""
    weights = n_layers * layer_params(c) + c.hidden_size + c.vocab_size * c.hidden_size
    weights += batch * c.hidden_size
    kv = kv_tokens * 2 * c.num_key_value_heads * c.head_dim * n_layers
    return (weights + kv) * elt


def prefill_flops(c, n_layers, t) -> float:
    """2 flops per weight and token in the layers, causal attention (half of the
    T x T scores and weighted sums), and the head for the one wanted row."""
    linear = 2.0 * t * n_layers * (layer_params(c) - 2 * c.hidden_size)
    attention = 2.0 * t * t * c.num_attention_heads * c.head_dim * n_layers
    head = 2.0 * c.vocab_size * c.hidden_size
    return linear + attention + head


class Families:
    """HIP events around every call of the kernel wrappers, by family, for one eager step.
    A call inside another measured call (a product that picks its kernel) counts once."""

    GEMM = ("linear", "gemm_bf16_skinny", "gemm_bf16_skinny_norm", "qkv_rope_append", "gemm_f32")
    ELEMENTWISE = ("rmsnorm", "silu_mul", "rope_append", "embedding", "residual_add")

    def __init__(self):
        self.spans = []
        self.depth = 0
        self.saved = []

    def _wrap(self, owner, name, family):
        import torch

        fn = getattr(owner, name)
        self.saved.append((owner, name, fn))

        def timed(*a, **kw):
            if self.depth:
                return fn(*a, **kw)
            self.depth += 1
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            try:
                return fn(*a, **kw)
            finally:
                end.record()
                self.depth -= 1
                self.spans.append((family, start, end))

        setattr(owner, name, timed)

    def __enter__(self):
        from halite_amd.kernels import attention as attention_kernels
        from halite_amd.kernels import ops

        for name in self.GEMM:
            self._wrap(ops, name, "gemm")
        for name in self.ELEMENTWISE:
            self._wrap(ops, name, "elementwise")
        self._wrap(attention_kernels, "paged_attention", "attention")
        return self

    def __exit__(self, *exc):
        for owner, name, fn in reversed(self.saved):
            setattr(owner, name, fn)
        self.saved = []

    def totals_ms(self) -> dict:
        import torch

        torch.cuda.synchronize()
        out = {}
        for family, start, end in self.spans:
            out[family] = out.get(family, 0.0) + start.elapsed_time(end)
        return out


def probe_gpu(torch) -> dict:
    """What this GPU gives the simplest streaming kernels and a large library product: a
    copy of 2 GiB (bytes read plus bytes written over time), a read of 2 GiB by the
    small-batch product with one row, and an 8192^3 bf16 product.  The rooflines above use the published peaks; these are the
    attainable ones."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.int16, device="cuda").fill_(1)
    dst = torch.empty_like(src)

    def best(fn, reps=5):
        times = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e-3)
        return min(times[1:])

    t_copy = best(lambda: dst.copy_(src))
    del dst
    # a pure read: one row against a 2 GiB bf16 matrix through the small-batch product
    from halite_amd.kernels import ops

    w = src.view(torch.bfloat16).view(-1, 4096)
    x = torch.zeros((1, 4096), dtype=torch.bfloat16, device="cuda")
    t_read = best(lambda: ops.gemm_bf16_skinny(x, w, out_dtype=torch.float32))
    del w
    m = 8192
    a = torch.randn((m, m), dtype=torch.bfloat16, device="cuda")
    b = torch.randn((m, m), dtype=torch.bfloat16, device="cuda")
    t_mm = best(lambda: torch.mm(a, b.t()))
    return {
        "copy_gbps": round(2 * 2 * n / t_copy / 1e9, 1),
        "read_gbps": round(2 * n / t_read / 1e9, 1),
        "gemm_8192_tflops": round(2.0 * m**3 / t_mm / 1e12, 1),
    }


def engine_workload(args) -> dict:
    """The two further workloads: requests through the scheduler (entry point, prompt
    portions, decoding, sampling); returns the record of one.

    ``mixed3b``: Llama-3.2-3B shape, 32 requests with prompt lengths uniform in 64..4096,
    prompts cut into portions of 512 tokens, 256 new tokens each.
    ``llama70b``: Llama-3.1-70B shape on the one GPU (141 GB of weights), 16 requests
    with 2,048-token prompts and 128 new tokens each.
    """
    import torch

    from halite_amd.config import LlamaConfig, ModelConfig, ServerConfig
    from halite_amd.engine.engine import InferenceEngine
    from halite_amd.engine.runner import ModelRunner
    from halite_amd.sampling import SamplingParams

    gen = torch.Generator().manual_seed(0)
    if args.workload == "mixed3b":
        raw, name = LLAMA_3_2_3B, "Llama-3.2-3B shape"
        lengths = torch.randint(64, 4097, (32,), generator=gen).tolist()
        new_tokens, chunk = 256, 512
    else:
        raw, name = LLAMA_3_1_70B, "Llama-3.1-70B shape"
        lengths, new_tokens, chunk = [2048] * 16, 128, 8192
    full = LlamaConfig(**raw)
    n_layers = args.layers or full.num_hidden_layers
    cfg = full.model_copy(update={"num_hidden_layers": n_layers})
    pool = sum(-(-(n + new_tokens) // 64) * 64 for n in lengths) + 1024
    server = ServerConfig(
        kv_cache_num_tokens=pool, max_seqs_per_forward=len(lengths), max_tokens_per_forward=8192,
        chunked_prefill_size=chunk, max_prefill_tokens=8192, use_cudagraph=not args.no_graph,
        cudagraph_max_batch_size=len(lengths), cudagraph_step=1, scheduling_steps_ahead=args.steps_ahead,
    )
    t0 = time.perf_counter()
    runner = ModelRunner.from_random(cfg, seed=0, server_config=server, model_config=ModelConfig(dtype=args.dtype, context_len=8192))
    torch.cuda.synchronize()
    print(f"[bench] {name}: {n_layers} layers built in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    engine = InferenceEngine(runner, None, seed=0)
    params = SamplingParams(max_new_tokens=new_tokens, temperature=0.0, ignore_eos=True)

    def requests():
        return [(torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist(), params) for n in lengths]

    # an untimed pass over a few short requests: libraries, graphs of the small batches
    engine.infer_batch([(torch.randint(0, cfg.vocab_size, (64,), generator=gen).tolist(),
                         SamplingParams(max_new_tokens=4, temperature=0.0, ignore_eos=True)) for _ in range(2)])
    engine.initialize(capture_graphs=not args.no_graph)  # as a server does before it takes requests
    graphs_before = len(runner._graphs)
    before = engine.stats.steps, engine.stats.retractions, len(engine.stats.tokens_per_step)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    results = engine.infer_batch(requests())
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    generated = sum(len(o) for r in results for o in r.output_ids)
    assert generated == len(lengths) * new_tokens, generated
    steps = engine.stats.steps - before[0]
    per_step = engine.stats.tokens_per_step[before[2]:]
    record = {
        "metric": f"generated tokens per second through the scheduler ({name}, {len(lengths)} requests)",
        "value": round(generated / dt, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": 0,
        "ms_per_step": round(dt / steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform-random token ids, random weights N(0, 0.02)",
        "config": {
            "model": name,
            "layers": n_layers,
            "layers_of_model": full.num_hidden_layers,
            "hidden_size": cfg.hidden_size,
            "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size,
            "vocab_size": cfg.vocab_size,
            "global_batch": len(lengths),
            "seq_len": max(lengths) + new_tokens,
            "prompt_tokens": sum(lengths),
            "new_tokens_each": new_tokens,
            "prefill_portion": chunk,
            "page_size": runner.cache.page_size,
            "hip_graph": not args.no_graph,
            "steps_ahead": args.steps_ahead,
            "parallelism": "single GPU",
        },
        "seconds": round(dt, 3),
        "total_tokens_per_second": round((generated + sum(lengths)) / dt, 1),
        "mean_tokens_per_step": round(sum(per_step) / max(1, len(per_step)), 1),
        "retractions": engine.stats.retractions - before[1],
        "steps_launched_ahead": engine.steps_launched_ahead,
        "graphs_recorded_before": graphs_before,
        "weights_gb": round(runner.model.param_bytes() / 1e9, 2),
    }
    del engine
    runner.release()
    return record


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=None, help="context length at the end of decoding")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration (named in the record)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--more-points", action="store_true",
                    help="further batches (16, 32, 128), contexts (32,768 and 131,072) and prompts (8,192 and 16,384)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel of a decode step from the host")
    ap.add_argument("--prefill-only", action="store_true", help="measure only the prefill (for profiles)")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="length of the prompt of the prefill measurement")
    ap.add_argument("--prefill-portion", type=int, default=0,
                    help="run the prompt of the prefill measurement in portions of this many tokens (0: whole)")
    ap.add_argument("--steps-ahead", type=int, default=1, choices=[0, 1],
                    help="launch a decode step before the tokens of the step before are read, as the engine does "
                         "by default (scheduling_steps_ahead); 0: read every step's tokens before the next is put together")
    ap.add_argument("--sampling", default="greedy", choices=["greedy", "temperature", "top_p", "top_k", "all"],
                    help="how the decode steps sample (the contract's line is greedy)")
    ap.add_argument("--workload", default="decode8b", choices=["decode8b", "mixed3b", "llama70b"],
                    help="decode8b: the headline line; the others run requests through the scheduler")
    ap.add_argument("--no-extras", action="store_true",
                    help="leave out what the default line adds beyond the contract's points: contexts of 32,768, "
                         "the 32-bit points and the 3B requests through the scheduler")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.workload != "decode8b":
        print(json.dumps(engine_workload(args)), flush=True)
        return 0

    import numpy as np
    import torch

    from halite_amd.config import LlamaConfig, ModelConfig, ServerConfig
    from halite_amd.engine.batch import Segment
    from halite_amd.engine.runner import ModelRunner
    from halite_amd.sampling import Sampler, SamplingParams

    full = LlamaConfig(**LLAMA_3_1_8B)
    n_layers = args.layers or full.num_hidden_layers
    cfg = full.model_copy(update={"num_hidden_layers": n_layers})
    context = args.context or 8192  # the benchmark's context; the model itself goes to 131,072
    dtype = args.dtype  # (the 32-bit points of the default line run the same functions once more)
    elt = 2 if dtype == "bfloat16" else 4
    extras = dtype == "bfloat16" and not (args.no_points or args.no_extras or args.prefill_only)
    LONG = 32768  # the further context of the default line
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    if args.dtype == "float32" and not args.no_points:
        batches = sorted({1, args.batch})  # the 32-bit path is for exactness: fewer, shorter points
    if args.prefill_only:
        batches, context = [1], max(4096, args.prefill_tokens + 64)
    # (batch, context at the end of decoding) of every point beyond the headline
    more = [(16, context), (32, context), (128, context), (8, 32768), (1, 131072), (8, 131072)] if args.more_points else []
    pool_tokens = max([b * (context + 64) for b in batches] + [b * (c + 64) for b, c in more]
                      + ([32 * (LONG + 64)] if extras else [])) + 4096
    longest = max([context] + [c for _, c in more] + ([16384 + 64] if args.more_points else []) + ([LONG + 64] if extras else []))
    runner = ModelRunner.from_random(
        cfg, seed=0,
        server_config=ServerConfig(kv_cache_num_tokens=pool_tokens,
                                   max_seqs_per_forward=max(batches + [b for b, _ in more] + ([32] if extras else [])) + 1,
                                   max_tokens_per_forward=16384, use_cudagraph=not args.no_graph,
                                   cudagraph_max_batch_size=max(batches + [b for b, _ in more] + ([32] if extras else []))),
        model_config=ModelConfig(dtype=dtype, context_len=longest),
    )
    sampler = Sampler(runner.device)
    greedy = SamplingParams(temperature=0.0)
    gen = torch.Generator().manual_seed(0)

    def sync():
        torch.cuda.synchronize()

    EXTRA_MARKED = 8

    def decode_run(batch: int, steps: int, warmup: int, end_context: int = context, families: bool = False,
                   keep: list | None = None, reuse: list | None = None):
        """Prefills ``batch`` prompts so that the contexts end at ``end_context`` after
        the last timed step, then times ``steps`` decode steps.  Returns the seconds, the
        mean number of cached tokens of a step, the GPU's share of the time (events around
        every step) and, if asked for, the families' times of one more, eager step.
        ``keep``: a list that takes the requests (slot, last token) instead of their being
        freed; ``reuse``: such requests, of which the first ``batch`` go on decoding from
        where they are (the others are freed) instead of new prompts."""
        prompt_len = end_context - steps - warmup - (2 + EXTRA_MARKED if families else 0)
        if reuse is not None:
            for s, _ in reuse[batch:]:
                runner.free(s)
            slots, last = [s for s, _ in reuse[:batch]], [t for _, t in reuse[:batch]]
        else:
            slots, last = [runner.admit() for _ in range(batch)], []
        t_said = time.perf_counter()
        for i_slot, s in enumerate(slots if reuse is None else []):
            if time.perf_counter() - t_said > 30:  # a long set-up says that it is alive
                sync()
                print(f"[bench] batch {batch}: prompt {i_slot} of {batch} ...", file=sys.stderr, flush=True)
                t_said = time.perf_counter()
            ids = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=gen).numpy().astype(np.int32)
            pos, tok = 0, None
            while pos < prompt_len:
                n = min(4096, prompt_len - pos)
                logits = runner.step([Segment(s, pos, ids[pos : pos + n], [n - 1] if pos + n == prompt_len else [])])
                pos += n
            tok, _ = sampler.forward(logits, [greedy], [0], [0])
            last.append(int(tok[0]))
        how = {"greedy": greedy, "temperature": SamplingParams(temperature=0.8),
               "top_p": SamplingParams(temperature=0.8, top_p=0.9), "top_k": SamplingParams(temperature=0.8, top_k=50),
               "all": SamplingParams(temperature=0.8, top_k=50, top_p=0.9, min_p=0.05)}[args.sampling]
        params, seeds, draws = [how] * batch, list(range(batch)), [0] * batch
        marks = []

        def one_step(tokens, mark=False):
            if mark:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
            segs = [Segment(s, runner.cache.length(s), [t], [0]) for s, t in zip(slots, tokens)]
            logits = runner.step(segs)
            toks, _ = sampler.forward(logits, params, seeds, draws)
            if mark:
                b.record()
                marks.append((a, b))
            return toks.tolist()

        def steps_launched_ahead(tokens, n):
            """``n`` steps as the engine runs them with ``scheduling_steps_ahead``: a step is
            launched with the tokens of the step before still on the device (its segments name
            their rows there), and the host reads a step's tokens while the next one runs."""
            feed = torch.tensor(tokens, dtype=torch.int32, device=runner.device)
            pinned, before = [torch.empty(batch, dtype=torch.int32, pin_memory=True) for _ in range(2)], None
            for i in range(n):
                segs = [Segment(s, runner.cache.length(s), [row], [0]) for row, s in enumerate(slots)]
                logits = runner.step(segs, token_feed=feed)
                feed, _ = sampler.forward(logits, params, seeds, draws)
                pinned[i % 2].copy_(feed, non_blocking=True)
                event = torch.cuda.Event()
                event.record()
                if before is not None:
                    before[1].synchronize()
                    tokens = before[0].tolist()
                before = (pinned[i % 2], event)
            before[1].synchronize()
            return before[0].tolist()

        if args.steps_ahead:
            last = steps_launched_ahead(last, warmup)
            sync()
            t0 = time.perf_counter()
            last = steps_launched_ahead(last, steps)
            sync()
            dt = time.perf_counter() - t0
        else:
            for _ in range(warmup):
                last = one_step(last)
            sync()
            t0 = time.perf_counter()
            for _ in range(steps):
                last = one_step(last)
            sync()
            dt = time.perf_counter() - t0
        gpu_s = None
        if families:
            # the GPU's share of a step: a few more steps with events around each (outside
            # the timed steps, which carry nothing extra)
            t1 = time.perf_counter()
            for _ in range(EXTRA_MARKED):
                last = one_step(last, mark=True)
            sync()
            gpu_s = (sum(a.elapsed_time(b) for a, b in marks) * 1e-3, time.perf_counter() - t1)
        kv_tokens = sum(runner.cache.length(s) for s in slots) - batch * (steps / 2.0 + (EXTRA_MARKED if families else 0))
        fam = None
        if families:
            # one more step, eager (every kernel launched from the host), with events
            # around every call of a kernel wrapper
            graph, runner.graphs_allowed = runner.graphs_allowed, False
            try:
                last = one_step(last)  # the eager path's first call (allocations, library loads)
                with Families() as f:
                    one_step(last)
                fam = f.totals_ms()
            finally:
                runner.graphs_allowed = graph
        if keep is not None:
            keep.extend(zip(slots, last))
        else:
            for s in slots:
                runner.free(s)
        return dt, kv_tokens, gpu_s, fam

    def prefill_run(T=args.prefill_tokens, families: bool = False, portion: int = 0):
        ids = torch.randint(0, cfg.vocab_size, (T,), generator=gen).numpy().astype(np.int32)
        times, fam = [], None
        for i in range(5 if families else 4):
            s = runner.admit()
            sync()
            measure = Families() if (families and i == 4) else None
            if measure:
                measure.__enter__()
            t0 = time.perf_counter()
            portion = portion or args.prefill_portion or T
            for start in range(0, T, portion):  # the whole prompt, or one portion a step
                end = min(start + portion, T)
                logits = runner.step([Segment(s, start, ids[start:end], [end - start - 1] if end == T else [])])
            tok, _ = sampler.forward(logits, [greedy], [0], [0])
            tok.tolist()
            sync()
            if measure:
                measure.__exit__()
                fam = measure.totals_ms()
            else:
                times.append(time.perf_counter() - t0)
            runner.free(s)
        t = min(times[1:])
        peak = PEAK_FLOPS["bf16" if dtype == "bfloat16" else "fp32"]
        out = {
            "value": round(T / t, 1),
            "tokens": T,
            "ms": round(t * 1e3, 3),
            "frac": round(prefill_flops(cfg, n_layers, T) / t / peak, 4),
        }
        if fam:
            linear = 2.0 * T * n_layers * (layer_params(cfg) - 2 * cfg.hidden_size) + 2.0 * cfg.vocab_size * cfg.hidden_size
            attention = 2.0 * T * T * cfg.num_attention_heads * cfg.head_dim * n_layers
            out["gemm_ms"] = round(fam.get("gemm", 0.0), 3)
            out["gemm_frac"] = round(linear / (fam["gemm"] * 1e-3) / peak, 4) if fam.get("gemm") else None
            out["attention_ms"] = round(fam.get("attention", 0.0), 3)
            out["attention_frac"] = round(attention / (fam["attention"] * 1e-3) / peak, 4) if fam.get("attention") else None
            out["elementwise_ms"] = round(fam.get("elementwise", 0.0), 3)
        return out

    if args.prefill_only:
        print(json.dumps({"metric": "prefill tokens per second", "layers": n_layers,
                          "prefill": prefill_run(families=True)}), flush=True)
        return 0

    # -- the headline: batch 8 -------------------------------------------------------
    results = {}
    for b in batches:
        steps = args.steps if b == args.batch else max(8, args.steps // 2)
        results[b] = (steps, *decode_run(b, steps, args.warmup, families=(b == args.batch)))
        print(f"[bench] decode batch {b}: {b * steps / results[b][1]:.1f} tok/s, "
              f"{results[b][1] / steps * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
    steps, dt, kv_tokens, gpu_s, fam = results[args.batch]
    value, step_s = args.batch * steps / dt, dt / steps
    need = decode_bytes(cfg, n_layers, args.batch, kv_tokens, elt)
    achieved = need / step_s

    def frac_of(batch, end_context, n_steps, seconds, cached):
        return round(decode_bytes(cfg, n_layers, batch, cached, elt) / (seconds / n_steps) / HBM_BYTES_PER_S, 4)

    record = {
        "metric": f"decode tokens per second (Llama-3.1-8B shape, batch {args.batch}, context {context})",
        "value": round(value, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform-random token ids, random weights N(0, 0.02)",
        "config": {
            "model": "Llama-3.1-8B shape",
            "layers": n_layers,
            "layers_of_model": full.num_hidden_layers,
            "hidden_size": cfg.hidden_size,
            "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size,
            "vocab_size": cfg.vocab_size,
            "global_batch": args.batch,
            "seq_len": context,
            "context_len": context,
            "prefill_tokens": args.prefill_tokens,
            "page_size": runner.cache.page_size,
            "hip_graph": not args.no_graph,
            "steps_ahead": args.steps_ahead,
            "sampling": args.sampling,
            "parallelism": "single GPU",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved / 1e9, 1),
            "peak": HBM_BYTES_PER_S / 1e9,
            "unit": "GB/s",
            "frac": round(achieved / HBM_BYTES_PER_S, 4),
        },
        # the step's wall time against the time the GPU works on it (events around every step)
    }
    if gpu_s:
        record["host"] = {"wall_ms": round(gpu_s[1] / EXTRA_MARKED * 1e3, 4), "gpu_ms": round(gpu_s[0] / EXTRA_MARKED * 1e3, 4),
                          "share": round(max(0.0, 1.0 - gpu_s[0] / gpu_s[1]), 4),
                          "how": f"{EXTRA_MARKED} further steps with HIP events around each, every step's tokens read before the next"}
    if fam:
        # one eager step with events around every kernel wrapper: the weight stream of the
        # products and the cache stream of attention, each against 8 TB/s
        weights = decode_bytes(cfg, n_layers, args.batch, 0, elt)
        cache = need - weights
        record["families"] = {
            "gemm": {"ms": round(fam.get("gemm", 0.0), 3), "frac": round(weights / (fam["gemm"] * 1e-3) / HBM_BYTES_PER_S, 4)},
            "attention": {"ms": round(fam.get("attention", 0.0), 3),
                          "frac": round(cache / (fam["attention"] * 1e-3) / HBM_BYTES_PER_S, 4)},
            "elementwise": {"ms": round(fam.get("elementwise", 0.0), 3)},
            "how": "one eager step, HIP events around each call",
        }

    if not args.no_points:
        points = {}
        for b in (1, 64):
            if b in results:
                n_steps, seconds, cached, _, _ = results[b]
                points[f"decode_b{b}"] = round(b * n_steps / seconds, 2)
                points[f"decode_b{b}_frac"] = frac_of(b, context, n_steps, seconds, cached)
        # the other reading of the decode points: prompts of 512 tokens, as the benchmark
        # configuration words its decode workload (the reference publishes no figures)
        for b in ((1, 8, 64) if dtype == "bfloat16" else (1, 8)):
            n_steps = max(8, args.steps // 2) if dtype == "bfloat16" else 4
            seconds, cached, _, _ = decode_run(b, n_steps, args.warmup, end_context=512 + n_steps + args.warmup)
            points[f"decode_p512_b{b}"] = round(b * n_steps / seconds, 2)
            points[f"decode_p512_b{b}_frac"] = frac_of(b, 0, n_steps, seconds, cached)
        for b, c in more:
            n_steps = max(8, args.steps // 4)
            seconds, cached, _, _ = decode_run(b, n_steps, 4, end_context=c)
            points[f"decode_b{b}_ctx{c}"] = round(b * n_steps / seconds, 2)
            points[f"decode_b{b}_ctx{c}_frac"] = frac_of(b, c, n_steps, seconds, cached)
            print(f"[bench] decode batch {b} context {c}: {points[f'decode_b{b}_ctx{c}']} tok/s", file=sys.stderr, flush=True)
        record["points"] = points
        record["prefill"] = prefill_run(families=True)
        if args.more_points:
            for T in (512, 8192, 16384):
                extra = prefill_run(T)
                points[f"prefill_{T}"] = extra["value"]
                points[f"prefill_{T}_frac"] = extra["frac"]
            # the default prompt in portions of 512 tokens, one a step (what a scheduler with
            # chunked_prefill_size=512 runs)
            extra = prefill_run(portion=512)
            points["prefill_in_portions_of_512"] = extra["value"]
            points["prefill_in_portions_of_512_frac"] = extra["frac"]
        record["probe"] = probe_gpu(torch)
        record["roofline"]["frac_of_measured_read"] = round(achieved / (record["probe"]["read_gbps"] * 1e9), 4)
        record["prefill"]["frac_of_measured_gemm"] = round(
            prefill_flops(cfg, n_layers, record["prefill"]["tokens"]) / (record["prefill"]["ms"] * 1e-3)
            / (record["probe"]["gemm_8192_tflops"] * 1e12), 4)
    if extras:
        # -- further sizes: 32 requests whose contexts end near 32,768, then 16 of them --
        t_extra = time.perf_counter()
        n_steps = max(8, args.steps // 4)
        held = []
        seconds, cached, _, _ = decode_run(32, n_steps, 4, end_context=LONG - n_steps - 4, keep=held)
        points[f"decode_b32_ctx{LONG}"] = round(32 * n_steps / seconds, 2)
        points[f"decode_b32_ctx{LONG}_frac"] = frac_of(32, LONG, n_steps, seconds, cached)
        seconds, cached, _, _ = decode_run(16, n_steps, 4, end_context=LONG, reuse=held)
        points[f"decode_b16_ctx{LONG}"] = round(16 * n_steps / seconds, 2)
        points[f"decode_b16_ctx{LONG}_frac"] = frac_of(16, LONG, n_steps, seconds, cached)
        extra = prefill_run(LONG)
        points[f"prefill_{LONG}"] = extra["value"]
        points[f"prefill_{LONG}_frac"] = extra["frac"]
        print(f"[bench] context {LONG}: decode batch 32 {points[f'decode_b32_ctx{LONG}']} tok/s, batch 16 "
              f"{points[f'decode_b16_ctx{LONG}']} tok/s, prefill {extra['value']} tok/s "
              f"({time.perf_counter() - t_extra:.0f} s)", file=sys.stderr, flush=True)
        # -- the 32-bit path: the same functions on a model of float32 --
        t_extra = time.perf_counter()
        runner.release()
        dtype, elt = "float32", 4
        runner = ModelRunner.from_random(
            cfg, seed=0,
            server_config=ServerConfig(kv_cache_num_tokens=args.batch * (context + 64) + 4096, max_seqs_per_forward=args.batch + 1,
                                       max_tokens_per_forward=16384, use_cudagraph=not args.no_graph,
                                       cudagraph_max_batch_size=args.batch),
            model_config=ModelConfig(dtype=dtype, context_len=context + 64),
        )
        n_steps = 8
        seconds, cached, _, _ = decode_run(args.batch, n_steps, 2)
        points[f"decode_b{args.batch}_fp32"] = round(args.batch * n_steps / seconds, 2)
        points[f"decode_b{args.batch}_fp32_ms"] = round(seconds / n_steps * 1e3, 3)
        points[f"decode_b{args.batch}_fp32_frac"] = frac_of(args.batch, context, n_steps, seconds, cached)
        extra = prefill_run()
        points[f"prefill_{extra['tokens']}_fp32"] = extra["value"]
        points[f"prefill_{extra['tokens']}_fp32_frac"] = extra["frac"]
        print(f"[bench] float32: decode batch {args.batch} {points[f'decode_b{args.batch}_fp32_ms']} ms/step, prefill "
              f"{extra['value']} tok/s ({time.perf_counter() - t_extra:.0f} s)", file=sys.stderr, flush=True)
        runner.release()
        dtype, elt = args.dtype, 2
        # -- requests through the scheduler: the 3B shape, 32 requests of mixed lengths --
        args.workload = "mixed3b"
        w = engine_workload(args)
        record["workloads"] = {"mixed3b": {
            "value": w["value"], "unit": "generated tok/s", "seconds": w["seconds"], "steps": w["steps"],
            "mean_tokens_per_step": w["mean_tokens_per_step"], "retractions": w["retractions"],
            "total_tokens_per_second": w["total_tokens_per_second"], "requests": w["config"]["global_batch"],
            "prompt_tokens": w["config"]["prompt_tokens"], "new_tokens_each": w["config"]["new_tokens_each"],
            "prefill_portion": w["config"]["prefill_portion"], "layers": w["config"]["layers"],
        }}
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
