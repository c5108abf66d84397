"""Grouped-query self-attention over the paged cache
(src/halite/transformers/infer/attention.py:20-172)."""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictInt, model_validator

from ..kernels import attention as attention_kernels
from ..kernels import ops
from .base import MIXERS, Mixer, PagedKVNeed, ParamDecl, RotaryPositionEncoding


class AttentionParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    n_kv_heads: StrictInt = Field(gt=0)
    head_dim: StrictInt = Field(gt=0)
    scale: float = Field(gt=0)
    position: str | None = None
    window: StrictInt | None = Field(default=None, gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.n_heads} heads are not a multiple of {self.n_kv_heads} kv heads")
        return self


@MIXERS.register("attention")
class Attention(Mixer):
    """q, k, v projections (separate weights, one packed tensor), rotation of q and
    k, append of k and v to the run's pages, attention of every token over the keys
    of its request up to itself (and no further back than ``window``), output
    projection.  Query head ``h`` reads key/value head ``h // (H/K)``.
    """

    Params = AttentionParams
    graph_safe = True
    takes_normed_rows = True
    folds_next_norm = True

    def __init__(self, params, build):
        super().__init__(params, build)
        self.position = None
        if params.position is not None:
            if params.position not in build.positions:
                raise ValueError(f"attention names position encoding {params.position!r}, which the model does not define")
            self.position = build.positions[params.position]
            if not isinstance(self.position, RotaryPositionEncoding):
                raise ValueError(
                    f"attention rotates queries and keys; position encoding {params.position!r} "
                    f"({type(self.position).__name__}) is not a RotaryPositionEncoding"
                )
            if self.position.rotary_dim > params.head_dim:
                raise ValueError("the position encoding rotates more elements than a head has")

    def param_decls(self):
        p = self.p
        return {
            "q.weight": ParamDecl((p.n_heads * p.head_dim, p.hidden_size)),
            "k.weight": ParamDecl((p.n_kv_heads * p.head_dim, p.hidden_size)),
            "v.weight": ParamDecl((p.n_kv_heads * p.head_dim, p.hidden_size)),
            "out.weight": ParamDecl((p.hidden_size, p.n_heads * p.head_dim)),
        }

    def allocate(self, dtypes):
        p = self.p
        if len({dtypes["q.weight"], dtypes["k.weight"], dtypes["v.weight"]}) != 1:
            raise ValueError("q, k and v weights are stored with different element types")
        nq, nk = p.n_heads * p.head_dim, p.n_kv_heads * p.head_dim
        dev = self.build.device
        self.w_qkv = torch.empty((nq + 2 * nk, p.hidden_size), dtype=dtypes["q.weight"], device=dev)
        self.w_out = torch.empty((p.hidden_size, nq), dtype=dtypes["out.weight"], device=dev)
        return {
            "q.weight": self.w_qkv[:nq],
            "k.weight": self.w_qkv[nq : nq + nk],
            "v.weight": self.w_qkv[nq + nk :],
            "out.weight": self.w_out,
        }

    def finalize(self):
        self.t_qkv = self.t_q = self.t_out = self.t_qkv_paired = None
        if self.build.tiled_weights and self.w_qkv.dtype == torch.bfloat16 and self.w_qkv.is_cuda:
            p = self.p
            self.t_out = ops.tile_weight(self.w_out) if self.w_out.dtype == torch.bfloat16 else None
            pos = self.position
            if (pos is not None and not pos.interleaved and pos.rotary_dim == p.head_dim
                    and p.head_dim % 16 == 0 and p.hidden_size % 8 == 0 and self.build.dtype == torch.bfloat16):
                # few tokens: projection, rotation and append are one kernel, which takes
                # the rows of a head in an order of its own
                self.t_qkv_paired = ops.tile_weight(ops.pair_rows_for_rotation(self.w_qkv, p.head_dim))
            else:
                self.t_qkv = ops.tile_weight(self.w_qkv)
                n_q = p.n_heads * p.head_dim
                if n_q % 16 == 0:  # the q rows are whole tiles at the front
                    steps = -(-p.hidden_size // 32)
                    self.t_q = self.t_qkv[: (n_q // 16) * steps * 512]

    def attention_sizes(self):
        return self.p.n_heads, self.p.n_kv_heads, self.p.head_dim

    def cache_need(self):
        return PagedKVNeed(self.p.n_kv_heads, self.p.head_dim, self.p.window)

    def prepare(self, ctx, run):
        group = ctx.cache.groups[run.kv.group_id]
        if attention_kernels.mfma_supported(self.build.dtype, self.p.head_dim, group.page_size):
            ctx.plan_attention(group.group_id, self.p.n_heads, self.p.n_kv_heads, self.p.window or 0, self.p.head_dim)

    def forward(self, x, ctx, run, then=None):
        p = self.p
        kv = run.kv
        group = ctx.group(kv.group_id)
        n_q = p.n_heads * p.head_dim
        if (run.appends and x.dtype == torch.bfloat16 and kv.k.dtype == torch.bfloat16
                and ops.norm_folds(x.shape[0], self.w_qkv.shape[0], x.shape[1], self.t_qkv_paired)):
            cos, sin = self.position.tables(ctx.max_position + 1)
            q = ops.qkv_rope_append(
                x, self.t_qkv_paired, ctx.positions, cos, sin, p.n_heads, p.n_kv_heads, p.head_dim,
                ctx.token_seg, group.block_table, kv.k, kv.v, group.page_size, kv.tiled,
            )
            out = ctx.attention(q, q.shape[1], kv, group, p.n_heads, p.scale, p.window or 0)
            return ops.linear(out, self.w_out, tiled=self.t_out, next_norm=then)
        if isinstance(x, ops.NormedRows):
            x = x.materialize()
        if run.appends:
            qkv = ops.linear(x, self.w_qkv, tiled=self.t_qkv)
            n_kv_append = p.n_kv_heads
        else:  # the keys and values are an earlier run's
            qkv = ops.linear(x, self.w_qkv[:n_q], tiled=self.t_q)
            n_kv_append = 0
        if self.position is not None:
            cos, sin = self.position.tables(ctx.max_position + 1)
            rot, interleaved = self.position.rotary_dim, self.position.interleaved
        else:
            cos = sin = ctx.empty_f32
            rot, interleaved = 0, False
        ops.rope_append(
            qkv, ctx.positions, cos, sin, p.n_heads, n_kv_append, p.head_dim, rot, interleaved,
            token_seg=ctx.token_seg, block_table=group.block_table,
            k_pages=kv.k, v_pages=kv.v, page_size=group.page_size, tiled=kv.tiled,
        )
        out = ctx.attention(qkv, qkv.shape[1], kv, group, p.n_heads, p.scale, p.window or 0)
        return ops.linear(out, self.w_out, tiled=self.t_out, next_norm=then)
