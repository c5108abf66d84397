"""The model: embedding, the layers in the order of the run list, final norm, head.

Built from a ``ModelSpec`` alone; which parts a layer has, in which arrangement, and
in which order the layers run are all data.  The flat-batch forward pass follows
src/halite/transformers/infer/transformer.py:82-114: embed, run every block on the
step's tokens, normalise the wanted rows, project them to float32 logits.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..config.spec import ModelSpec
from .base import (
    ARRANGEMENTS,
    EMBEDDINGS,
    HEADS,
    NORMS,
    POSITIONS,
    BuildContext,
    ConfigError,
    ParamDecl,
    Part,
    RunBinding,
)


@dataclass
class ParamSlot:
    path: str  # e.g. layers.3.mixer.q.weight
    part: Part
    name: str  # the part's own name for it, e.g. q.weight
    decl: ParamDecl


class Decoder:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device: torch.device | str,
                 tiled_weights: bool = False):
        # the kinds of parts register themselves when their modules are imported
        from . import attention, block, embedding, feedforward, norm, rope  # noqa: F401

        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        build = BuildContext(dtype=dtype, device=self.device, hidden_size=spec.hidden_size,
                             tiled_weights=tiled_weights and dtype == torch.bfloat16)
        for name, pspec in spec.positions.items():
            build.positions[name] = POSITIONS.build(pspec, build)
        self.build = build
        self.positions = build.positions
        self.embedding = EMBEDDINGS.build(spec.embedding, build)
        self.layers = {}
        for name, lspec in spec.layers.items():
            if lspec.arrangement not in ARRANGEMENTS:
                known = ", ".join(sorted(ARRANGEMENTS))
                raise ConfigError(f"unknown arrangement {lspec.arrangement!r}; known: {known}")
            self.layers[name] = ARRANGEMENTS[lspec.arrangement].build(lspec.arrangement, lspec.parts, build)
        self.final_norm = NORMS.build(spec.final_norm, build)
        self.head = HEADS.build(spec.head, build)
        self.runs = [
            RunBinding(index=i, appends=run.cache_from is None) for i, run in enumerate(spec.order)
        ]

    # -- declarations -------------------------------------------------------------
    def named_parts(self) -> dict[str, Part]:
        out = {"embedding": self.embedding}
        for lname, block in self.layers.items():
            for pname, part in block.parts().items():
                out[f"layers.{lname}.{pname}"] = part
        out["final_norm"] = self.final_norm
        out["head"] = self.head
        return out

    def param_slots(self) -> list[ParamSlot]:
        """Every tensor of the model in a fixed order (the order that the random
        weights are drawn in)."""
        slots = []
        for prefix, part in self.named_parts().items():
            for name, decl in part.param_decls().items():
                slots.append(ParamSlot(f"{prefix}.{name}", part, name, decl))
        return slots

    def mixer_of_run(self, index: int):
        return self.layers[self.spec.order[index].layer].mixer

    def finalize(self):
        self.head.bind(self.embedding)
        for part in self.named_parts().values():
            part.finalize()

    def param_bytes(self) -> int:
        n = 0
        for slot in self.param_slots():
            size = 1
            for d in slot.decl.shape:
                size *= d
            n += size * (4 if slot.decl.integer else self.dtype.itemsize)
        return n

    # -- the forward pass of one step -----------------------------------------------
    def forward(self, ctx) -> torch.Tensor:
        """float32 logits ``[len(ctx.logit_rows), vocab]``; keys and values of all
        the step's tokens are in the cache afterwards."""
        h = self.embedding.forward(ctx.tokens)
        pending = None
        blocks = [self.layers[self.spec.order[run.index].layer] for run in self.runs]
        for i, run in enumerate(self.runs):
            # what the next block's first norm lets this block's last product do for it
            # (both are optional abilities of an arrangement: `takes_next_norm` of the one that
            # runs now, `first_norm_for` of the one that runs next)
            ahead = blocks[i + 1] if i + 1 < len(blocks) else None
            next_norm = None
            if getattr(blocks[i], "takes_next_norm", False) and hasattr(ahead, "first_norm_for"):
                next_norm = ahead.first_norm_for(h)
            if next_norm is not None:
                pending = blocks[i].forward(h, pending, ctx, run, next_norm=next_norm)
            else:
                pending = blocks[i].forward(h, pending, ctx, run)
        if ctx.n_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        x = self.final_norm.forward(h, delta=pending, rows=ctx.logit_rows)
        return self.head.forward(x)
