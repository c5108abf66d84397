"""Generate tokens from a model folder.

In the manner of the reference's scripts (scripts/eval_task.py:161-185): ``--model``
names the checkpoint folder, and free ``key=value`` words after the options override
fields of the configuration objects: ``sampling.<field>`` (SamplingParams),
``server.<field>`` (ServerConfig) and ``model.<field>`` (ModelConfig), e.g.

    python -m halite_amd.cli.generate --model DIR --prompt-ids 1,2,3 \\
        sampling.temperature=0.8 sampling.max_new_tokens=24 server.page_size=16

Instead of ``--model``, ``--random CONFIG.json`` (with ``--weights-seed``) runs a model of
that configuration with seeded random weights, drawn on the device and never written.

Prompts are token ids (``--prompt-ids``, repeatable; ``--prompt-file`` with one JSON
list a line) or seeded uniform-random ids of given lengths (``--prompt-lens``).
Results are printed as one JSON object a line.
"""

from __future__ import annotations

import argparse
import json
import sys

import torch

from ..config import ModelConfig, ServerConfig, parse_overrides, read_config


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", type=str, help="folder with config.json and model.safetensors")
    ap.add_argument("--random", type=str, metavar="CONFIG.json",
                    help="instead of --model: a config.json whose model gets seeded random weights N(0, 0.02)")
    ap.add_argument("--weights-seed", type=int, default=0, help="seed of the random weights of --random")
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; repeatable")
    ap.add_argument("--prompt-file", type=str, help="file with one JSON list of token ids a line")
    ap.add_argument("--prompt-lens", type=str, help="comma-separated lengths of random prompts")
    ap.add_argument("--prompt-seed", type=int, default=0)
    ap.add_argument("--seed", type=int, default=0, help="engine seed for sampling streams")
    ap.add_argument("--stats", action="store_true", help="print scheduler statistics to stderr")
    ap.add_argument("opts", default=[], nargs="*", help="key=value overrides")
    return ap.parse_intermixed_args(argv)  # overrides and options in any order


def split_overrides(opts):
    groups = {"sampling": {}, "server": {}, "model": {}}
    for key, value in parse_overrides([o for o in (opts or []) if o != "--"]).items():
        head, _, field = key.partition(".")
        if head not in groups or not field:
            raise SystemExit(f"override {key!r}: use sampling.<field>, server.<field> or model.<field>")
        groups[head][field] = value
    return groups


def main(argv=None) -> int:
    """Runs ``generate`` and turns what a user can get wrong (a folder, an option, a
    request) into one line on stderr and exit status 2."""
    from ..config.registry import ConfigError
    from ..weights import WeightError

    args = parse_args(argv)
    try:
        return generate(args)
    except (ConfigError, WeightError, ValueError, TypeError, FileNotFoundError) as e:
        print(f"halite_generate: error: {e}", file=sys.stderr)
        return 2


def generate(args) -> int:
    over = split_overrides(args.opts)
    from ..engine import InferenceEngine
    from ..sampling import SamplingParams

    if bool(args.model) == bool(args.random):
        raise SystemExit("give one of --model DIR and --random CONFIG.json")
    if args.random:
        from ..config import parse_config

        with open(args.random) as f:
            arch, cfg = parse_config(json.load(f))
    else:
        arch, cfg = read_config(args.model)
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [json.loads(line) for line in f if line.strip()]
    if args.prompt_lens:
        gen = torch.Generator().manual_seed(args.prompt_seed)
        vocab_size = arch.to_spec(cfg).vocab_size  # (the configuration's own key for it is the architecture's business)
        for n in args.prompt_lens.split(","):
            prompts.append(torch.randint(0, vocab_size, (int(n),), generator=gen).tolist())
    if not prompts:
        raise SystemExit("no prompts: give --prompt-ids, --prompt-file or --prompt-lens")

    server, model = ServerConfig(**over["server"]), ModelConfig(**over["model"])
    if args.random:
        from ..engine.runner import ModelRunner

        engine = InferenceEngine(ModelRunner.from_random(cfg, args.weights_seed, server, model), None, seed=args.seed)
    else:
        engine = InferenceEngine.from_pretrained(args.model, server, model, seed=args.seed)
    params = SamplingParams(**over["sampling"])
    results = engine.infer_batch([(i, p, params) for i, p in enumerate(prompts)])
    for r in results:
        print(json.dumps(r.to_dict()))
    if args.stats:
        s = engine.stats
        print(
            f"steps {s.steps} prefill tokens {s.prefill_tokens} decode tokens {s.decode_tokens} "
            f"retractions {s.retractions} elapsed {engine.last_elapsed:.3f} s",
            file=sys.stderr,
        )
    return 0


if __name__ == "__main__":
    sys.exit(main())
