"""Write a model folder with seeded random weights.

The counterpart of the reference's checkpoint tool (scripts/tools/
convert_checkpoint.py:27-85: ``--conf`` and ``--out``): ``--config`` is a
``config.json`` of the architecture, ``--out`` the folder that receives
``config.json`` and ``model.safetensors``.
"""

from __future__ import annotations

import argparse
import json
import sys

from ..config import parse_config
from ..weights import write_random_model


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--config", required=True, help="a config.json")
    ap.add_argument("--out", required=True)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dtype", choices=["float32", "bfloat16"], default="bfloat16")
    ap.add_argument("--std", type=float, default=0.02)
    args = ap.parse_args(argv)
    with open(args.config) as f:
        arch, cfg = parse_config(json.load(f))
    write_random_model(args.out, cfg, args.seed, args.dtype, args.std, arch)
    print(args.out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
