"""RMSNorm (src/halite/nn/normalization.py:13-57)."""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictInt

from ..kernels import ops
from .base import NORMS, Norm, ParamDecl


class RMSNormParams(BaseModel):
    size: StrictInt = Field(gt=0)
    eps: float = Field(gt=0)


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """``weight * (x * rsqrt(mean(x^2) + eps))``: statistics and scaling in float32,
    the normalised value rounded to the activation type before the weight
    multiplies it (normalization.py:48-55).  The residual add that precedes the
    norm in a block (src/halite/transformers/block.py:56-74) is fused in."""

    Params = RMSNormParams
    graph_safe = True

    def param_decls(self):
        return {"weight": ParamDecl((self.p.size,), init="ones")}

    def forward(self, h, delta=None, rows=None):
        if isinstance(delta, ops.NormedRows):
            # the product before has added its result into h and prepared these rows
            if delta.weight is not self.weight or rows is not None:
                raise ValueError("rows were prepared for another norm")
            return delta
        return ops.rmsnorm(h, self.weight, self.p.eps, self.build.dtype, delta=delta, rows=rows)

    def foldable(self, h):
        if self.build.dtype != torch.bfloat16 or not h.is_cuda:
            return None
        return ops.NextNorm(h, self.weight, self.p.eps)
