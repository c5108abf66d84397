"""Layers of the Llama-3.1-8B shape against the plain implementation, in 32-bit and in
bfloat16, under the four ways of cutting the work (each request whole; the last 32 tokens
one by one; portions of changing size; mixed with other requests on few pages), with
bounds that the figures must meet.

The whole depth is not collected by pytest (32 layers need about 70 GB of host memory and
some minutes); run it as

    python tests/full_depth_equality.py [--layers 32] [--out FILE]

It exits with 1 if a bound is missed.  ``tests/test_replay_gpu.py`` runs the same check
with 8 layers.

Weights N(0, 0.02) are drawn once on the CPU and handed to the plain implementation (a dict
in memory) and to the engine (``load_state_dict``).  The bounds, relative to the largest
logit of a request:

* float32: every row of every schedule within 1e-4 of the plain implementation.
* bfloat16: the yardstick is the plain implementation with ``round_to=torch.bfloat16`` (the
  results of products, rotation, attention, activation and norms rounded; statistics,
  softmax and residual in float32), whose distance from float32 arithmetic on the same
  (rounded) weights is what the number format costs at this depth: ``E``, and ``R`` for the
  root mean square.  The engine may lie no further from float32 arithmetic than 1.3 E (and
  1.3 R), and no further from the rounding implementation than 1.5 E (1.5 R): two
  computations that round at the same places but add in another order drift apart like two
  independent ones, by about the square root of two times the error of each.
"""

import argparse
import gc
import os
import sys
import time

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import plain_llama  # noqa: E402
import replay  # noqa: E402
import tiny  # noqa: E402
from halite_amd.config import ModelConfig, ServerConfig, parse_config  # noqa: E402
from halite_amd.engine.runner import ModelRunner  # noqa: E402

LLAMA_8B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256, num_hidden_layers=32,
    rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)
SCHEDULES = {"whole": replay.whole, "last 32 one by one": replay.tail_one_by_one,
             "portions": replay.portions, "mixed": replay.mixed}
FLOAT32_BOUND = 1e-4
FROM_FLOAT32 = 1.3  # bfloat16 engine against float32 arithmetic, in units of the rounding implementation's own distance
FROM_ROUNDING = 1.5  # bfloat16 engine against the rounding implementation, in the same units


def distance(rows: dict, ref: dict) -> tuple[float, float, int]:
    """Largest |difference| of a row over its request's largest |logit| (at least 1); root
    mean square of the differences over that of the reference; rows compared."""
    worst = sq = ref_sq = 0.0
    n = 0
    for rid, by_pos in rows.items():
        scale = max(1.0, float(ref[rid].abs().max()))
        for p, row in by_pos.items():
            d = row - ref[rid][p]
            err = float(d.abs().max()) / scale
            if err != err:
                raise AssertionError(f"request {rid} position {p}: NaN in the logits")
            worst = max(worst, err)
            sq += float((d**2).sum())
            ref_sq += float((ref[rid][p] ** 2).sum())
            n += 1
    return worst, (sq / ref_sq) ** 0.5, n


def all_rows(ref: dict) -> dict:
    return {rid: {p: t[p] for p in range(t.shape[0])} for rid, t in ref.items()}


def run(layers: int, lengths, say=lambda *a: None, command: str = ""):
    """The check itself: (lines of a summary, list of missed bounds)."""
    raw = dict(LLAMA_8B, num_hidden_layers=layers)
    _, cfg = parse_config(raw)
    weights = tiny.random_weights(raw, seed=11, std=0.02)
    say("weights drawn")
    requests = {f"r{i}": tiny.random_tokens(raw, int(n), 70 + i) for i, n in enumerate(lengths)}
    lines = [
        f"# {layers} layers of the Llama-3.1-8B shape against the plain implementation",
        "",
        f"Command: `{command}`" if command else "",
        "",
        f"Weights N(0, 0.02), norm weights 1 ± 0.1; requests of {', '.join(map(str, lengths))} tokens; every position's",
        "logits compared.  'largest' is the largest |difference| of a logit row over the request's largest |logit|,",
        "'rms' the root mean square of the differences over that of the logits.",
        "",
        "| precision | schedule | steps | rows | against | largest | rms | bound on largest | met |",
        "|---|---|---:|---:|---|---:|---:|---:|---|",
    ]
    missed = []

    def judge(dtype, name, trace, n, against, worst, rms, bound, rms_bound=None):
        ok = worst <= bound and (rms_bound is None or rms <= rms_bound)
        lines.append(f"| {dtype} | {name} | {len(trace)} | {n} | {against} | {worst:.2e} | {rms:.2e} | {bound:.2e} | {'yes' if ok else 'NO'} |")
        if not ok:
            missed.append(f"{dtype}, {name}, against {against}: largest {worst:.3e} (bound {bound:.3e}), rms {rms:.3e}"
                          + (f" (bound {rms_bound:.3e})" if rms_bound is not None else ""))

    for dtype in ("float32", "bfloat16"):
        if dtype == "bfloat16":
            for k in list(weights):
                weights[k] = weights[k].to(torch.bfloat16).float()
            say("weights rounded to bfloat16")
        ref = {rid: plain_llama.forward(raw, weights, toks) for rid, toks in requests.items()}
        say(dtype, "plain forward done")
        rounding = e_fmt = r_fmt = None
        if dtype == "bfloat16":
            rounding = {rid: plain_llama.forward(raw, weights, toks, round_to=torch.bfloat16) for rid, toks in requests.items()}
            e_fmt, r_fmt, n = distance(all_rows(rounding), ref)
            say(f"rounding implementation against float32 arithmetic: largest {e_fmt:.3e}, rms {r_fmt:.3e}")
            lines.append(f"| bfloat16 | (the plain implementation rounding to bfloat16) | | {n} | float32 arithmetic | {e_fmt:.2e} | {r_fmt:.2e} | | |")
        for name, make in SCHEDULES.items():
            trace = make(requests)
            server = ServerConfig(kv_cache_num_tokens=replay.peak_tokens(trace), page_size=64, max_seqs_per_forward=8)
            runner = ModelRunner.from_random(cfg, 0, server, ModelConfig(dtype=dtype))
            runner.load_state_dict(weights)
            rows = replay.collect(trace, replay.run_trace(runner, trace), raw["vocab_size"])
            worst, rms, n = distance(rows, ref)
            if dtype == "float32":
                judge(dtype, name, trace, n, "plain implementation", worst, rms, FLOAT32_BOUND)
            else:
                judge(dtype, name, trace, n, "float32 arithmetic", worst, rms, FROM_FLOAT32 * e_fmt, FROM_FLOAT32 * r_fmt)
                w2, r2, _ = distance(rows, rounding)
                judge(dtype, name, trace, n, "rounding implementation", w2, r2, FROM_ROUNDING * e_fmt, FROM_ROUNDING * r_fmt)
            say(dtype, name, f"largest difference {worst:.3e}")
            runner.release()
            del runner
            gc.collect()
            torch.cuda.empty_cache()
    return lines, missed


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--lengths", default="70,9,150,33")
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    t0 = time.time()

    def say(*a):
        print(f"[{time.time() - t0:6.1f}s]", *a, file=sys.stderr, flush=True)

    command = f"python tests/full_depth_equality.py --layers {args.layers} --lengths {args.lengths}"
    lines, missed = run(args.layers, [int(n) for n in args.lengths.split(",")], say, command)
    lines += ["", "Bounds missed: " + ("none" if not missed else "")] + [f"* {m}" for m in missed]
    text = "\n".join(lines) + "\n"
    print(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text)
    return 1 if missed else 0


if __name__ == "__main__":
    sys.exit(main())
