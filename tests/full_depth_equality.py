"""All layers of the Llama-3.1-8B shape against the plain implementation, in 32-bit and in
bfloat16, under the four ways of cutting the work (each request whole; the last 32 tokens
one by one; portions of changing size; mixed with other requests on few pages).

Not collected by pytest (it needs about 70 GB of host memory and some minutes): run it as

    python tests/full_depth_equality.py [--layers 32] [--out FILE]

It draws weights N(0, 0.02) once on the CPU, hands the same tensors to the plain
implementation (a dict in memory) and to the engine (``load_state_dict``), replays the
schedules through ``ModelRunner`` and prints, per precision and schedule, the largest
difference of any logit row from the plain implementation's, relative to the largest
logit.  In bfloat16 the plain implementation computes in float32 on the weights rounded
to bfloat16, so the figure there is the rounding of activations through all layers.
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--lengths", default="70,9,150,33")
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    t0 = time.time()

    def say(*a):
        print(f"[{time.time() - t0:6.1f}s]", *a, file=sys.stderr, flush=True)

    raw = dict(LLAMA_8B, num_hidden_layers=args.layers)
    _, cfg = parse_config(raw)
    weights = tiny.random_weights(raw, seed=11, std=0.02)
    say("weights drawn")
    requests = {f"r{i}": tiny.random_tokens(raw, int(n), 70 + i) for i, n in enumerate(args.lengths.split(","))}
    lines = [
        f"# {args.layers} layers of the Llama-3.1-8B shape against the plain implementation",
        "",
        f"Command: `python tests/full_depth_equality.py --layers {args.layers} --lengths {args.lengths}`",
        "",
        f"Weights N(0, 0.02), norm weights 1 ± 0.1; requests of {args.lengths} tokens; every position's logits",
        "compared; figures are the largest |difference| of a logit row divided by the largest |logit|.",
        "",
        "| precision | schedule | steps | rows compared | largest difference | rms difference / rms logit |",
        "|---|---|---:|---:|---:|---:|",
    ]
    for dtype in ("float32", "bfloat16"):
        if dtype == "bfloat16":
            for k in list(weights):
                weights[k] = weights[k].to(torch.bfloat16).float()
            say("weights rounded to bfloat16")
        ref = {rid: plain_llama.forward(raw, weights, toks) for rid, toks in requests.items()}
        say(dtype, "plain forward done")
        for name, make in SCHEDULES.items():
            trace = make(requests)
            server = ServerConfig(kv_cache_num_tokens=replay.peak_tokens(trace), page_size=64, max_seqs_per_forward=8)
            runner = ModelRunner.from_random(cfg, 0, server, ModelConfig(dtype=dtype))
            runner.load_state_dict(weights)
            rows = replay.collect(trace, replay.run_trace(runner, trace), raw["vocab_size"])
            worst = replay.compare(rows, ref, 1.0)
            sq = n = 0.0
            ref_sq = 0.0
            for rid, by_pos in rows.items():
                for p, row in by_pos.items():
                    sq += float(((row - ref[rid][p]) ** 2).sum())
                    ref_sq += float((ref[rid][p] ** 2).sum())
                    n += 1
            lines.append(f"| {dtype} | {name} | {len(trace)} | {int(n)} | {worst:.2e} | {(sq / ref_sq) ** 0.5:.2e} |")
            say(dtype, name, f"largest difference {worst:.3e}")
            runner.release()
            del runner
            gc.collect()
            torch.cuda.empty_cache()
    text = "\n".join(lines) + "\n"
    print(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text)


if __name__ == "__main__":
    main()
