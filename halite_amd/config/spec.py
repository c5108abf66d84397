"""The description of a model as data: parts, layers and the order they run in.

The reference composes its module tree at configuration time from numbers
(configs/models/transformer.py:55-311: ``build_block`` takes the norm, the
attention, the feed-forward and the position encoding as arguments) and
serialises that tree to plain dicts.  This is the same idea with typed nodes:
a ``ModelSpec`` is plain data that round-trips through JSON, every part is named
by ``kind`` and carries all its sizes and constants, and the order in which
layers run is a list of its own, so a layer can run twice or read the cache that
an earlier run wrote.
"""

from __future__ import annotations

from typing import Any

from pydantic import BaseModel, ConfigDict, StrictInt, model_validator


class PartSpec(BaseModel):
    """One part: ``kind`` picks the class from the part registry, the other
    keys are that class's own parameters (validated by the class)."""

    model_config = ConfigDict(extra="allow")

    kind: str

    def params(self) -> dict[str, Any]:
        return {k: v for k, v in self.model_dump().items() if k != "kind"}


class LayerSpec(BaseModel):
    """A block: which arrangement, and the parts that the arrangement asks for, by the
    names it gives them (src/halite/transformers/block.py:10-85 takes its norms, its
    attention and its feed-forward as arguments in the same way).  Which names exist, and
    which of them may be left out, is the arrangement's to say: ``pre_norm`` has
    ``mixer_norm``, ``mixer``, ``ff_norm`` and ``ff``.  A name the arrangement does not
    know is an error when the model is built, never dropped."""

    model_config = ConfigDict(extra="forbid")

    arrangement: str = "pre_norm"
    parts: dict[str, PartSpec]

    @model_validator(mode="before")
    @classmethod
    def _parts_as_keywords(cls, data):
        """``LayerSpec(mixer=..., ff=...)`` stands for ``LayerSpec(parts={"mixer": ..., "ff": ...})``."""
        if isinstance(data, dict) and "parts" not in data:
            data = dict(data)
            head = {"arrangement": data.pop("arrangement")} if "arrangement" in data else {}
            data = {**head, "parts": data}
        return data


class LayerRun(BaseModel):
    """One entry of the run order.

    ``layer`` names an entry of ``ModelSpec.layers`` (the weights).  Every run
    has a cache of its own unless ``cache_from`` gives the index of an earlier
    run: then the mixer appends nothing and reads that run's cache.
    """

    layer: str
    cache_from: StrictInt | None = None


class ModelSpec(BaseModel):
    architecture: str
    vocab_size: StrictInt
    hidden_size: StrictInt
    max_positions: StrictInt
    embedding: PartSpec
    positions: dict[str, PartSpec]
    layers: dict[str, LayerSpec]
    order: list[LayerRun]
    final_norm: PartSpec
    head: PartSpec

    @model_validator(mode="after")
    def _check(self):
        for i, run in enumerate(self.order):
            if run.layer not in self.layers:
                raise ValueError(f"order[{i}] names unknown layer {run.layer!r}")
            if run.cache_from is not None:
                if not 0 <= run.cache_from < i:
                    raise ValueError(
                        f"order[{i}].cache_from={run.cache_from} must name an earlier run"
                    )
                if self.order[run.cache_from].cache_from is not None:
                    raise ValueError(
                        f"order[{i}].cache_from={run.cache_from} names a run that owns no cache"
                    )
        return self
