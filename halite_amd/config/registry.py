"""One registry from an architecture's name to what builds its model.

The reference chooses the architecture by the configuration file that is loaded
and swaps training classes for inference classes with a patch list
(configs/models/transformer.py:314-430).  Here the name in ``config.json``
(``architectures[0]``) picks an ``Architecture``: its typed configuration, the
function that turns the configuration into a ``ModelSpec`` and the table that maps
tensor names of the folder to parameters of the parts.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable

from pydantic import BaseModel, ValidationError

from .spec import ModelSpec


class ConfigError(ValueError):
    pass


@dataclass(frozen=True)
class Architecture:
    """What the framework asks of an architecture.

    ``config_cls`` is a pydantic model of the architecture's ``config.json``.  Beside its
    own keys it must have the field ``architectures`` (a list whose first entry is
    ``name``: what a model folder is recognised by, and what the random-weights mode
    writes).  It may have ``stop_token_ids`` (token ids that end a request unless it asks
    to ignore them) and a method ``to_json_dict()`` (the ``config.json`` to write, if
    ``model_dump(exclude_none=True)`` is not it).  Nothing else of it is read outside
    ``to_spec`` and ``weight_map``, which are the architecture's own."""

    name: str
    config_cls: type[BaseModel]
    to_spec: Callable[[BaseModel], ModelSpec]
    # pattern of a tensor name in the folder -> parameter path in the model;
    # '#' stands for a layer name (configs/models/llama/checkpoint.py:94-158)
    weight_map: Callable[[BaseModel], dict[str, str]]


ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> Architecture:
    fields = getattr(arch.config_cls, "model_fields", None)
    if fields is None or "architectures" not in fields:
        raise ConfigError(
            f"architecture {arch.name!r}: its configuration class must be a pydantic model with "
            "the field 'architectures'"
        )
    for optional in ("to_json_dict",):
        if hasattr(arch.config_cls, optional) and not callable(getattr(arch.config_cls, optional)):
            raise ConfigError(f"architecture {arch.name!r}: {optional} of its configuration class is not a method")
    ARCHITECTURES[arch.name] = arch
    return arch


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    if name not in ARCHITECTURES:
        known = ", ".join(sorted(ARCHITECTURES)) or "(none)"
        raise ConfigError(f"unknown architecture {name!r}; known: {known}")
    return ARCHITECTURES[name]


def _load_builtin():
    from .. import architectures  # noqa: F401  (registers on import)


def parse_config(raw: dict) -> tuple[Architecture, BaseModel]:
    names = raw.get("architectures")
    if not names or not isinstance(names, list):
        raise ConfigError("config.json has no 'architectures' list")
    arch = get_architecture(names[0])
    try:
        cfg = arch.config_cls(**raw)
    except ValidationError as e:
        raise ConfigError(f"config.json is not a valid {arch.name} configuration:\n{e}") from e
    return arch, cfg


def read_config(folder: str) -> tuple[Architecture, BaseModel]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder}: no config.json")
    with open(path) as f:
        raw = json.load(f)
    return parse_config(raw)
