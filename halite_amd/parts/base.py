"""What every part of a model is, and the registries that hold the kinds of parts.

A part (mixer, feed-forward, norm, position encoding, embedding, head) is built from
its own validated parameters and a ``BuildContext``; it declares the tensors it owns,
what cache and what fixed-size per-request state it needs, and computes on the tokens
of one step.  No part knows which model it is in: the reference composes its blocks
the same way from interchangeable modules (configs/models/transformer.py:55-196).

Registering a new kind is one decorator; the model builder looks kinds up by the
``kind`` string of a ``PartSpec``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Any, ClassVar

import torch
from pydantic import BaseModel, ValidationError

from ..config.registry import ConfigError
from ..config.spec import PartSpec

if TYPE_CHECKING:
    from ..engine.batch import StepContext


@dataclass(frozen=True)
class ParamDecl:
    """A tensor that a part owns.  ``init`` is what the random-weights mode does
    with it: ``normal`` (N(0, std) from the seed) or ``ones``."""

    shape: tuple[int, ...]
    init: str = "normal"
    integer: bool = False


class PagedNeed:
    """Something of every token, kept in pages.  What a mixer's ``cache_need`` returns is a
    frozen dataclass of this kind: runs whose needs are equal share one group of pages (one
    block table per request for all of them).  The cache manager reads three things of a need:

    * ``window`` (an attribute; ``None``: every token's page is kept while the request lives;
      else the tokens a query looks back, itself included, so that pages are given back once
      every later query has passed them);
    * ``page_tensors(page_size)``: name -> shape of one page, the tensors a run keeps per page
      number, all of the cache's element type;
    * ``bind(group_id, tensors, page_size, dtype)``: what the run's mixer finds in ``run.kv``,
      made of those tensors (each ``[pages, *shape]``).
    """

    window: int | None = None

    def page_tensors(self, page_size: int) -> dict[str, tuple[int, ...]]:
        raise NotImplementedError

    def bind(self, group_id: int, tensors: dict[str, torch.Tensor | None], page_size: int, dtype: torch.dtype):
        raise NotImplementedError


@dataclass(frozen=True)
class PagedKVNeed(PagedNeed):
    """Keys and values of every token: keys ``[K, page_size, D]`` and values, transposed,
    ``[K, D, page_size]`` per page (or the same bytes in the matrix-core attention kernel's
    order, see ``cache.pages.tiled_layout``); ``run.kv`` is a ``cache.pages.LayerPages``."""

    n_kv_heads: int
    head_dim: int
    window: int | None = None

    def page_tensors(self, page_size: int) -> dict[str, tuple[int, ...]]:
        k, d = self.n_kv_heads, self.head_dim
        return {"k": (k, page_size, d), "v": (k, d, page_size)}

    def bind(self, group_id, tensors, page_size, dtype):
        from ..cache.pages import LayerPages, tiled_layout

        return LayerPages(group_id, tensors["k"], tensors["v"], tiled_layout(dtype, self.head_dim, page_size))


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size that a request keeps between steps, one row per live
    request, zero when the request is admitted."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class BuildContext:
    dtype: torch.dtype  # element type of activations and cache
    device: torch.device
    hidden_size: int
    positions: dict[str, "Part"] = field(default_factory=dict)
    # keep a second copy of every bf16 matrix in the small-batch kernel's tiled order
    tiled_weights: bool = False


@dataclass
class RunBinding:
    """What one entry of the run order is bound to at run time."""

    index: int
    kv: Any = None  # cache.pages.LayerPages of this run (own or borrowed), or None
    appends: bool = True  # False: the cache belongs to an earlier run
    state: dict[str, torch.Tensor] = field(default_factory=dict)  # [n_slots, *shape]


class Part:
    """Base of all parts."""

    Params: ClassVar[type[BaseModel]]
    # True: what ``forward`` launches depends only on how many tokens each segment of the
    # step has and how many rows are wanted; everything else (token ids, positions, pages,
    # slots, lengths of the contexts) it reads on the device, from the step's arrays.  A
    # step recorded into a graph can then be replayed for another step of that shape.  A
    # model is run from graphs only if all of its parts say so.
    graph_safe: ClassVar[bool] = False

    def __init__(self, params: BaseModel, build: BuildContext):
        self.p = params
        self.build = build

    # -- declarations ---------------------------------------------------------
    def param_decls(self) -> dict[str, ParamDecl]:
        return {}

    def allocate(self, dtypes: dict[str, torch.dtype]) -> dict[str, torch.Tensor]:
        """Creates the part's tensors on the device with the given element types
        and returns, for every name of ``param_decls``, the tensor (or the view
        into a packed tensor) that the loader fills.  The default makes one
        attribute per name (``q.weight`` becomes ``self.q_weight``)."""
        out = {}
        for name, decl in self.param_decls().items():
            t = torch.empty(decl.shape, dtype=dtypes[name], device=self.build.device)
            setattr(self, name.replace(".", "_"), t)
            out[name] = t
        return out

    def finalize(self) -> None:
        """Called once after the tensors are filled."""

    def cache_need(self) -> PagedNeed | None:
        return None

    def state_need(self) -> dict[str, StateNeed]:
        return {}


class Mixer(Part):
    """Mixes information between the tokens of a request (attention here).

    Two optional abilities, which a block uses only where both neighbours have them (so a
    part without them never sees either): ``takes_normed_rows``, ``forward`` accepts
    ``kernels.ops.NormedRows`` for ``x`` (rows whose norm the part's first product
    finishes); ``folds_next_norm``, ``forward`` takes ``then=ops.NextNorm`` and may
    return ``NormedRows`` for that norm, with its result already added into the stream,
    instead of the result."""

    takes_normed_rows: ClassVar[bool] = False
    folds_next_norm: ClassVar[bool] = False

    def attention_sizes(self) -> tuple[int, int, int] | None:
        """(query heads, key/value heads, head size) if the mixer has such sizes, for the
        check of sizes that a caller states beside the model (``ModelConfig.n_heads`` and
        its like); None if it has none."""
        return None

    def prepare(self, ctx: "StepContext", run: RunBinding) -> None:
        """Called for every run before the step's arrays go to the device; a mixer
        may add host-built arrays of its own to that one copy."""

    def forward(self, x: torch.Tensor, ctx: "StepContext", run: RunBinding) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    # as for Mixer
    takes_normed_rows: ClassVar[bool] = False
    folds_next_norm: ClassVar[bool] = False

    def forward(self, x: torch.Tensor, ctx: "StepContext") -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    def forward(
        self,
        h: torch.Tensor,
        delta: torch.Tensor | None = None,
        rows: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """Normalises the float32 stream ``h`` after adding ``delta`` to it (the sum
        is written back to ``h``); with ``rows`` only those rows, and ``h`` is left
        as it is.  ``delta`` may be what a product left for this norm
        (``kernels.ops.NormedRows``, see ``foldable``), which is handed on as it is."""
        raise NotImplementedError

    def foldable(self, h: torch.Tensor):
        """``kernels.ops.NextNorm`` if the product before this norm may add into ``h`` and
        prepare the norm's input itself, else None."""
        return None


class PositionEncoding(Part):
    """Says where a token is.  What a position encoding offers is for the mixers that name it
    to use; the one contract the framework's own mixers know is ``RotaryPositionEncoding``."""


class RotaryPositionEncoding(PositionEncoding):
    """A position encoding that is applied by rotating pairs of the first ``rotary_dim``
    elements of every query and key head: pairs ``(j, j + rotary_dim/2)``, or neighbours
    ``(2j, 2j + 1)`` if ``interleaved``."""

    @property
    def rotary_dim(self) -> int:
        raise NotImplementedError

    @property
    def interleaved(self) -> bool:
        raise NotImplementedError

    def tables(self, n_positions: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """float32 ``(cos, sin)``, each ``[at least n_positions, rotary_dim / 2]``, on the
        device; row ``p`` holds the angles of position ``p``."""
        raise NotImplementedError


class Embedding(Part):
    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    def bind(self, embedding: "Embedding") -> None:
        """Called once, before ``finalize``, with the model's embedding: a head that shares
        tensors with it (tied weights) takes them here."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Registry:
    def __init__(self, what: str):
        self.what = what
        self.kinds: dict[str, type[Part]] = {}

    def register(self, kind: str):
        def deco(cls):
            self.kinds[kind] = cls
            cls.kind = kind
            return cls

        return deco

    def build(self, spec: PartSpec, build: BuildContext) -> Part:
        if spec.kind not in self.kinds:
            known = ", ".join(sorted(self.kinds)) or "(none)"
            raise ConfigError(f"unknown {self.what} kind {spec.kind!r}; known: {known}")
        cls = self.kinds[spec.kind]
        try:
            params = cls.Params(**spec.params())
        except ValidationError as e:
            raise ConfigError(f"{self.what} {spec.kind!r}: bad parameters:\n{e}") from e
        return cls(params, build)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("head")
class Arrangement:
    """The order in which a layer's parts act on the residual stream.

    ``roles``: name of a part -> the registry its kind is looked up in; ``optional``:
    names that a layer may leave out (the arrangement then finds ``None`` under them).
    ``forward(h, pending, ctx, run)`` gets the float32 stream ``h`` [tokens, width], a
    delta ``pending`` that the block before has not added yet (or ``None``), the step and
    the run's binding; it adds into ``h`` what it adds and returns the delta it leaves to
    whoever comes next (or ``None``).  Every arrangement has a part named ``mixer``."""

    roles: ClassVar[dict[str, "Registry"]] = {}
    optional: ClassVar[tuple[str, ...]] = ()
    graph_safe: ClassVar[bool] = False  # as for Part

    def __init__(self, parts: dict[str, Part | None]):
        self._parts = dict(parts)
        self.mixer = parts["mixer"]

    def parts(self) -> dict[str, Part]:
        """The parts that exist, by name (their tensors are ``layers.<layer>.<name>.*``)."""
        return {name: part for name, part in self._parts.items() if part is not None}

    def forward(self, h, pending, ctx, run):
        raise NotImplementedError

    @classmethod
    def build(cls, kind: str, specs: dict[str, PartSpec], build: BuildContext) -> "Arrangement":
        if "mixer" not in cls.roles:
            raise ConfigError(f"arrangement {kind!r} declares no part named 'mixer'")
        unknown = sorted(set(specs) - set(cls.roles))
        missing = sorted(set(cls.roles) - set(specs) - set(cls.optional))
        if unknown or missing:
            raise ConfigError(
                f"arrangement {kind!r} is made of {sorted(cls.roles)}"
                + (f"; it has no part named {unknown}" if unknown else "")
                + (f"; the layer leaves out {missing}" if missing else "")
            )
        return cls({name: (reg.build(specs[name], build) if name in specs else None)
                    for name, reg in cls.roles.items()})


ARRANGEMENTS: dict[str, type[Arrangement]] = {}


def register_arrangement(kind: str):
    def deco(cls):
        ARRANGEMENTS[kind] = cls
        return cls

    return deco
