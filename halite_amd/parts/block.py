"""How the parts of a layer are arranged (src/halite/transformers/block.py:10-85).

An arrangement says which parts it is made of, by name and by kind of part
(``roles``), which of them may be left out (``optional``), and how a step's tokens
go through them.  The builder makes the parts that the layer's description names,
refuses names that the arrangement does not have, and hands the arrangement a dict.
One part of every arrangement is its ``mixer``: the part that may own a cache and
per-request state, which the step function binds to every run of the layer.
"""

from __future__ import annotations

from .base import FEED_FORWARDS, MIXERS, NORMS, Arrangement, register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock(Arrangement):
    """``h = h + mixer(norm(h)); h = h + ff(norm(h))`` (block.py:56-74).

    The residual stream ``h`` is float32.  Each add is done by the norm that
    follows it, so the block hands its last delta on to the next block's first
    norm (or to the model's final norm) instead of adding it itself.
    """

    graph_safe = True
    roles = {"mixer_norm": NORMS, "mixer": MIXERS, "ff_norm": NORMS, "ff": FEED_FORWARDS}
    takes_next_norm = True  # forward() accepts next_norm=

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer_norm, self.ff_norm, self.ff = parts["mixer_norm"], parts["ff_norm"], parts["ff"]

    # The norm between two parts can be folded into the products around it where the part
    # before it offers that and the part after it takes such rows.
    def first_norm_for(self, h):
        """For the block that runs before this one: what its last product may prepare."""
        return self.mixer_norm.foldable(h) if self.mixer.takes_normed_rows else None

    def forward(self, h, pending, ctx, run, next_norm=None):
        x = self.mixer_norm.forward(h, delta=pending)
        then = None
        if self.mixer.folds_next_norm and self.ff.takes_normed_rows:
            then = self.ff_norm.foldable(h)
        a = self.mixer.forward(x, ctx, run, then=then) if then is not None else self.mixer.forward(x, ctx, run)
        x = self.ff_norm.forward(h, delta=a)
        if next_norm is not None and self.ff.folds_next_norm:
            return self.ff.forward(x, ctx, then=next_norm)
        return self.ff.forward(x, ctx)
