"""The random-weights mode.

``write_random_model`` makes a model folder (``config.json`` and
``model.safetensors`` under the architecture's own tensor names) from a
configuration and a seed; ``fill_random`` draws the same kind of weights straight
into a model on the device, for sizes that nobody wants to write to disk.  Matrices
and tables are N(0, std), norm weights are 1, as the benchmark configurations
prescribe; the reference's own initialiser is a training one
(src/halite/transformers/transformer.py:92-108; src/halite/nn/normalization.py:33-41
for the ones).

Every tensor has a generator of its own, seeded from (seed, position of the tensor
in the model's fixed order), so tensors can be made one at a time.
"""

from __future__ import annotations

import json
import os

import torch

from ..config.registry import Architecture, get_architecture
from ..parts.decoder import Decoder
from .loader import expand_weight_map
from .safetensors_io import SafetensorsWriter

_STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _tensor_seed(seed: int, index: int) -> int:
    return (seed * 1_000_003 + index * 7919 + 1) % (2**63 - 1)


def _draw(decl, seed: int, index: int, std: float, device, dtype) -> torch.Tensor:
    if decl.init == "ones":
        return torch.ones(decl.shape, dtype=dtype, device=device)
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, index))
    t = torch.randn(decl.shape, generator=gen, dtype=torch.float32, device=device) * std
    return t.to(dtype)


def write_random_model(folder: str, cfg, seed: int, dtype: str = "float32", std: float = 0.02,
                       arch: Architecture | None = None) -> str:
    """Writes ``folder/config.json`` and ``folder/model.safetensors``; the tensors
    are drawn on the CPU in float32 and stored as ``dtype``."""
    arch = arch or get_architecture(cfg.architectures[0])
    store = _STORE[dtype]
    os.makedirs(folder, exist_ok=True)
    model = Decoder(arch.to_spec(cfg), store, "cpu")
    name_of = {v: k for k, v in expand_weight_map(arch.weight_map(cfg), list(model.spec.layers)).items()}
    slots = model.param_slots()
    layout = [(name_of[s.path], torch.int32 if s.decl.integer else store, tuple(s.decl.shape)) for s in slots]
    writer = SafetensorsWriter(os.path.join(folder, "model.safetensors"), layout, {"format": "pt"})
    for i, s in enumerate(slots):
        writer.write(name_of[s.path], _draw(s.decl, seed, i, std, "cpu", store))
    writer.close()
    raw = cfg.to_json_dict() if hasattr(cfg, "to_json_dict") else cfg.model_dump(exclude_none=True)
    raw["torch_dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f, indent=2)
    return folder


def fill_random(model: Decoder, seed: int, std: float = 0.02) -> None:
    """Allocates the model's tensors in its own element type and fills them on the
    device (values differ from ``write_random_model``'s, whose generator is the
    CPU's)."""
    slots = model.param_slots()
    by_part: dict[int, dict[str, torch.dtype]] = {}
    for s in slots:
        by_part.setdefault(id(s.part), {})[s.name] = torch.int32 if s.decl.integer else model.dtype
    views = {}
    for s in slots:
        if id(s.part) not in views:
            views[id(s.part)] = s.part.allocate(by_part[id(s.part)])
    for i, s in enumerate(slots):
        dst = views[id(s.part)][s.name]
        dst.copy_(_draw(s.decl, seed, i, std, model.device, dst.dtype))
    model.finalize()
