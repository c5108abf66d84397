"""Token embedding and output head (src/halite/transformers/embedding.py:7-51;
src/halite/transformers/feedforward.py:72-114)."""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Embedding, Head, ParamDecl


class EmbeddingParams(BaseModel):
    vocab_size: StrictInt = Field(gt=0)
    size: StrictInt = Field(gt=0)


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Embedding):
    """Row lookup without a multiplier (embedding.py:36-44) into the float32
    residual stream."""

    Params = EmbeddingParams
    graph_safe = True

    def param_decls(self):
        return {"weight": ParamDecl((self.p.vocab_size, self.p.size))}

    def forward(self, tokens):
        return ops.embedding(tokens, self.weight)


class LinearHeadParams(BaseModel):
    vocab_size: StrictInt = Field(gt=0)
    size: StrictInt = Field(gt=0)
    tied: StrictBool = False


@HEADS.register("linear_head")
class LinearHead(Head):
    """Bias-free projection to the vocabulary with float32 logits
    (src/halite/transformers/infer/postprocessor.py:45-57).  When ``tied`` the
    weight is the embedding's table itself
    (src/halite/transformers/transformer.py:59-61), bound by the model builder."""

    Params = LinearHeadParams
    graph_safe = True

    def param_decls(self):
        if self.p.tied:
            return {}
        return {"weight": ParamDecl((self.p.vocab_size, self.p.size))}

    def bind(self, embedding):
        if self.p.tied:
            self.weight = embedding.weight

    def finalize(self):
        self.t_weight = None
        if self.build.tiled_weights and self.weight.dtype == torch.bfloat16 and self.weight.is_cuda:
            self.t_weight = ops.tile_weight(self.weight)

    def forward(self, x):
        return ops.linear(x, self.weight, out_dtype=torch.float32, tiled=self.t_weight)
