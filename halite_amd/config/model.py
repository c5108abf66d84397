"""Typed configuration of the Llama 3 decoder, read from its own ``config.json`` keys.

The reference validates model sizes with a strict pydantic schema
(src/halite/transformers/config.py:4-14) and passes every other constant into
its builder functions as an argument (configs/models/transformer.py:55-81,
201-311).  Here the schema is the architecture's ``config.json``; nothing the
file gives has a default in code except options whose absence has a meaning
(no ``rope_scaling`` means unscaled frequencies, no ``num_key_value_heads`` means
one key/value head per query head as in configs/models/transformer.py:115-116).
"""

from __future__ import annotations

from typing import Literal

from pydantic import BaseModel, ConfigDict, Field, StrictBool, StrictInt, model_validator


class Llama3RopeScaling(BaseModel):
    """Arguments of the Llama 3 frequency scaling,
    src/halite/transformers/position.py:242-284."""

    model_config = ConfigDict(extra="ignore")

    rope_type: Literal["llama3"]
    factor: float = Field(gt=0)
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: StrictInt = Field(gt=0)

    @model_validator(mode="before")
    @classmethod
    def _accept_old_key(cls, data):
        if isinstance(data, dict) and "rope_type" not in data and "type" in data:
            data = dict(data)
            data["rope_type"] = data["type"]
        return data

    @model_validator(mode="after")
    def _check(self):
        if self.high_freq_factor == self.low_freq_factor:
            raise ValueError("rope_scaling: high_freq_factor equals low_freq_factor")
        return self


class LlamaConfig(BaseModel):
    """``config.json`` of a ``LlamaForCausalLM`` folder."""

    model_config = ConfigDict(extra="ignore")

    architectures: list[str] = ["LlamaForCausalLM"]
    vocab_size: StrictInt = Field(gt=0)
    hidden_size: StrictInt = Field(gt=0)
    num_hidden_layers: StrictInt = Field(gt=0)
    num_attention_heads: StrictInt = Field(gt=0)
    num_key_value_heads: StrictInt | None = Field(default=None, gt=0)
    head_dim: StrictInt | None = Field(default=None, gt=0)
    intermediate_size: StrictInt = Field(gt=0)
    rms_norm_eps: float = Field(gt=0)
    rope_theta: float = Field(gt=0)
    rope_scaling: Llama3RopeScaling | None = None
    # False: pairs are (j, j + D/2), the layout q_proj/k_proj rows of such a
    # folder are stored for (position.py:287-291).  True: adjacent pairs
    # (2j, 2j+1), the reference's own Llama choice for Meta-format weights
    # (position.py:294-300, configs/models/llama/llama3_2_3b.py:18).
    rope_interleaved: StrictBool = False
    max_position_embeddings: StrictInt = Field(gt=0)
    tie_word_embeddings: StrictBool = False
    attention_bias: StrictBool = False
    mlp_bias: StrictBool = False
    hidden_act: str = "silu"
    torch_dtype: str | None = None
    bos_token_id: int | list[int] | None = None
    eos_token_id: int | list[int] | None = None

    @model_validator(mode="before")
    @classmethod
    def _accept_other_spellings(cls, data):
        """Folders written by newer tools carry ``rope_parameters`` (the base and the
        scaling arguments in one dict) instead of ``rope_theta`` and ``rope_scaling``,
        and may name the unscaled frequencies ``"default"``."""
        if not isinstance(data, dict):
            return data
        data = dict(data)
        merged = data.get("rope_parameters")
        if isinstance(merged, dict):
            if "rope_theta" not in data and "rope_theta" in merged:
                data["rope_theta"] = merged["rope_theta"]
            if "rope_scaling" not in data:
                data["rope_scaling"] = {k: v for k, v in merged.items() if k != "rope_theta"}
        scaling = data.get("rope_scaling")
        if isinstance(scaling, dict) and scaling.get("rope_type", scaling.get("type")) == "default":
            data["rope_scaling"] = None
        return data

    @model_validator(mode="after")
    def _check(self):
        if self.num_key_value_heads is None:
            self.num_key_value_heads = self.num_attention_heads
        if self.head_dim is None:
            if self.hidden_size % self.num_attention_heads:
                raise ValueError(
                    f"hidden_size {self.hidden_size} is not a multiple of "
                    f"num_attention_heads {self.num_attention_heads} and no head_dim is given"
                )
            self.head_dim = self.hidden_size // self.num_attention_heads
        if self.num_attention_heads % self.num_key_value_heads:
            raise ValueError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}"
            )
        if self.head_dim % 2:
            raise ValueError(f"head_dim {self.head_dim} is odd: rotation needs pairs")
        if self.attention_bias or self.mlp_bias:
            raise ValueError("Llama 3 has no biases (attention_bias / mlp_bias must be false)")
        if self.hidden_act != "silu":
            raise ValueError(f"hidden_act {self.hidden_act!r}: Llama 3 uses 'silu'")
        return self

    @property
    def stop_token_ids(self) -> tuple[int, ...]:
        eos = self.eos_token_id
        if eos is None:
            return ()
        return tuple(eos) if isinstance(eos, list) else (eos,)

    def to_json_dict(self) -> dict:
        """The dict that is written as ``config.json`` (round-trips through
        ``LlamaConfig(**d)``)."""
        d = self.model_dump(exclude_none=True)
        if not self.rope_interleaved:
            d.pop("rope_interleaved")
        return d
