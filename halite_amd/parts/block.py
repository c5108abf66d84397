"""How the parts of a layer are arranged (src/halite/transformers/block.py:10-85)."""

from __future__ import annotations

from .base import register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock:
    """``h = h + mixer(norm(h)); h = h + ff(norm(h))`` (block.py:56-74).

    The residual stream ``h`` is float32.  Each add is done by the norm that
    follows it, so the block hands its last delta on to the next block's first
    norm (or to the model's final norm) instead of adding it itself.
    """

    def __init__(self, mixer_norm, mixer, ff_norm, ff):
        self.mixer_norm, self.mixer, self.ff_norm, self.ff = mixer_norm, mixer, ff_norm, ff

    def parts(self):
        return {
            "mixer_norm": self.mixer_norm,
            "mixer": self.mixer,
            "ff_norm": self.ff_norm,
            "ff": self.ff,
        }

    def forward(self, h, pending, ctx, run):
        x = self.mixer_norm.forward(h, delta=pending)
        a = self.mixer.forward(x, ctx, run)
        x = self.ff_norm.forward(h, delta=a)
        return self.ff.forward(x, ctx)
