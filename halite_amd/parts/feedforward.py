"""The gated feed-forward (src/halite/transformers/feedforward.py:175-225)."""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictInt, field_validator

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamDecl


class GatedParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    intermediate_size: StrictInt = Field(gt=0)
    activation: str = "silu"

    @field_validator("activation")
    @classmethod
    def _known(cls, v):
        if v != "silu":
            raise ValueError(f"activation {v!r}: only 'silu' has a kernel")
        return v


@FEED_FORWARDS.register("gated")
class GatedFeedForward(FeedForward):
    """``linear_out(linear_proj(x) * silu(linear_gate(x)))`` without biases
    (feedforward.py:204-212).  Gate and up weights live in one tensor
    ``[2F, d]`` (gate first) so that one product serves both; the activation and
    the multiply are float32 on the accumulators or on the product's output."""

    Params = GatedParams
    graph_safe = True
    takes_normed_rows = True
    folds_next_norm = True

    def param_decls(self):
        f, d = self.p.intermediate_size, self.p.hidden_size
        return {
            "linear_gate.weight": ParamDecl((f, d)),
            "linear_proj.weight": ParamDecl((f, d)),
            "linear_out.weight": ParamDecl((d, f)),
        }

    def allocate(self, dtypes):
        f, d = self.p.intermediate_size, self.p.hidden_size
        dev = self.build.device
        if dtypes["linear_gate.weight"] != dtypes["linear_proj.weight"]:
            raise ValueError("gate and up weights are stored with different element types")
        self.w_gate_up = torch.empty((2 * f, d), dtype=dtypes["linear_gate.weight"], device=dev)
        self.w_out = torch.empty((d, f), dtype=dtypes["linear_out.weight"], device=dev)
        return {
            "linear_gate.weight": self.w_gate_up[:f],
            "linear_proj.weight": self.w_gate_up[f:],
            "linear_out.weight": self.w_out,
        }

    def finalize(self):
        self.t_gate = self.t_up = self.t_out = None
        f = self.p.intermediate_size
        if self.build.tiled_weights and self.w_gate_up.is_cuda:
            if self.w_gate_up.dtype == torch.bfloat16:
                self.t_gate = ops.tile_weight(self.w_gate_up[:f])
                self.t_up = ops.tile_weight(self.w_gate_up[f:])
            if self.w_out.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.w_out)

    def forward(self, x, ctx, then=None):
        f = self.p.intermediate_size
        w = self.w_gate_up
        # The gated product with SiLU·mul in its epilogue beats the library product and a
        # kernel for SiLU·mul up to 16 rows, and at 17 to 32 rows on matrices of up to 64 M
        # elements (measured in captured graphs: 50 against 56 us at 14336 x 4096, 23 against
        # 25 at 8192 x 3072, 202 against 179 at 28672 x 8192).
        m, d = x.shape
        small = (self.t_gate is not None and x.dtype == torch.bfloat16 and d % 8 == 0
                 and (m <= ops.SKINNY_ROWS or (m <= ops.FUSED_ROWS and f * d <= ops.GATED_MID_ELEMENTS)))
        if isinstance(x, ops.NormedRows):
            if small:
                act = ops.gemm_bf16_skinny_norm(x, self.t_gate, (f, d), w_up_tiled=self.t_up)
                return ops.linear(act, self.w_out, tiled=self.t_out, next_norm=then)
            x = x.materialize()
        if small:
            act = ops.gemm_bf16_skinny(x, self.t_gate, w_up=self.t_up, tiled_shape=(f, d))
            return ops.linear(act, self.w_out, tiled=self.t_out, next_norm=then)
        fused = (
            w.dtype == torch.bfloat16
            and x.dtype == torch.bfloat16
            and ops.skinny_pays(x.shape[0], f, x.shape[1], False)
            and x.shape[1] % 8 == 0
            and (f * x.shape[1]) % 8 == 0
        )
        if fused:
            act = ops.gemm_bf16_skinny(x, w[:f], w_up=w[f:])
        else:
            act = ops.silu_mul(ops.linear(x, w))
        return ops.linear(act, self.w_out, tiled=self.t_out, next_norm=then)
