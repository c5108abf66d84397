"""Options of the engine, under the reference's names where it has them.

``ServerConfig`` takes the scheduler knobs of the reference's ``infer`` engine
(src/halite/transformers/infer/types.py:67-81) and the paging and per-step limits of
its ``tokainfer`` engine (src/halite/transformers/tokainfer/types.py:65-190);
``ModelConfig`` keeps what src/halite/transformers/infer/types.py:84-113 holds beyond
the sizes that the model's own configuration already gives.
"""

from __future__ import annotations

from typing import Literal

from pydantic import BaseModel, ConfigDict, Field, StrictBool, StrictInt


class ServerConfig(BaseModel):
    model_config = ConfigDict(extra="forbid")

    # -- infer/types.py:67-81 ------------------------------------------------
    max_prefill_tokens: StrictInt = Field(default=16384, gt=0)
    """Most prompt tokens that one step may hold."""
    chunked_prefill_size: StrictInt = Field(default=8192, gt=0)
    """Most tokens of one prompt in one step; longer prompts are cut into portions."""
    default_init_new_token_ratio: float = 0.7
    default_min_new_token_ratio_factor: float = 0.14
    default_new_token_ratio_decay_steps: StrictInt = 600
    schedule_conservativeness: float = 1.0
    use_cudagraph: StrictBool = False
    """Replay decode-only steps from a captured HIP graph."""
    cudagraph_max_batch_size: StrictInt = 64
    """Largest decode batch that is replayed from a graph.  A graph here serves the batch
    size it was recorded for and nothing is padded (the reference pads a batch up to the
    next size it has a graph for, model_runner.py:160-166), so every size up to this one
    gets a graph of its own, at its first use or ahead of time."""
    cudagraph_step: StrictInt = Field(default=16, gt=0)
    cudagraph_additonal_batch_size: tuple[StrictInt, ...] = ()
    """The sizes whose graphs are recorded ahead of time
    (``InferenceEngine.initialize(capture_graphs=True)``): the additional ones and every
    multiple of the step up to the largest, as the reference lists its graph sizes
    (model_runner.py:86-95; the option's name is spelled as there).  Other sizes are
    recorded when a step first has them."""

    # -- tokainfer/types.py:65-190 -------------------------------------------
    page_size: StrictInt = Field(default=64, gt=0)
    kv_cache_num_tokens: StrictInt | None = Field(default=None, gt=0)
    """Tokens the cache pool holds; ``None`` sizes it from free device memory
    with ``memory_fraction_static`` (infer/engine/model_runner.py:117-131)."""
    max_tokens_per_forward: StrictInt = Field(default=8192, gt=0)
    """Token budget of one step: decoded tokens plus prompt portions."""
    max_seqs_per_forward: StrictInt = Field(default=256, gt=0)
    """Most requests that are live (own a slot) at a time."""

    scheduling_steps_ahead: StrictInt = Field(default=0, ge=0, le=1)
    """1: a decode step is launched before the tokens of the step before it have been
    read; they reach it on the device (the reference's second engine schedules ahead
    too, tokainfer/types.py:99).  A request that turns out to have stopped leaves
    one unused row behind."""

    # -- ours -----------------------------------------------------------------
    decode_weight_copy: Literal["auto", "on", "off"] = "auto"
    """A second copy of the bf16 matrices in the small-batch kernel's tiled order
    (steps of up to 16 tokens then read contiguous memory).  ``auto`` keeps it when
    two copies of the weights take less than a third of the device's memory."""

    # -- retraction (infer/engine/batch.py:468-527) ----------------------------
    retract_decode_steps: StrictInt = Field(default=20, gt=0)


class ModelConfig(BaseModel):
    """Run-time options of the model (infer/types.py:84-113).  The sizes that the
    reference repeats here (heads, layers) come from the model's configuration."""

    model_config = ConfigDict(extra="forbid")

    context_len: StrictInt | None = Field(default=None, gt=0)
    """Longest request; ``None`` takes the model's ``max_position_embeddings``."""
    n_heads: StrictInt | None = Field(default=None, gt=0)
    n_key_value_heads: StrictInt | None = Field(default=None, gt=0)
    head_dim: StrictInt | None = Field(default=None, gt=0)
    n_layers: StrictInt | None = Field(default=None, gt=0)
    """The reference's engine is told these (infer/types.py:85-89, scripts/eval_task.py:148-154);
    here the model says them, and what a caller states is only checked against it."""
    tp_size: Literal[1] = 1
    distributed: Literal[False] = False
    dtype: Literal["bfloat16", "float32"] = "bfloat16"
    kv_cache_dtype: Literal["auto"] = "auto"
    memory_fraction_static: float = Field(default=0.88, gt=0, le=1)
    gpu_id: StrictInt = 0
    device: str = "cuda"


def check_stated_sizes(options: ModelConfig, n_layers: int, attention_sizes: list[tuple[int, int, int]]) -> None:
    """Raises if sizes that a caller states in ``options`` (as the reference's callers do)
    disagree with the model: ``n_layers`` runs, and ``(heads, key/value heads, head size)``
    of every layer that has them."""
    wrong = []
    if options.n_layers is not None and options.n_layers != n_layers:
        wrong.append(f"n_layers={options.n_layers} (the model runs {n_layers})")
    for name, at in (("n_heads", 0), ("n_key_value_heads", 1), ("head_dim", 2)):
        stated = getattr(options, name)
        have = sorted({sizes[at] for sizes in attention_sizes})
        if stated is not None and have != [stated]:
            wrong.append(f"{name}={stated} (the model's layers have {', '.join(map(str, have)) or 'none'})")
    if wrong:
        raise ValueError("model options disagree with the model: " + "; ".join(wrong))


def parse_overrides(pairs: list[str]) -> dict:
    """``key=value`` command-line overrides (the reference's
    ``apply_overrides``, scripts/eval_task.py:179-182) as a dict of strings
    that pydantic then validates and converts."""
    import json

    out = {}
    for pair in pairs:
        if "=" not in pair:
            raise ValueError(f"override {pair!r} is not of the form key=value")
        key, value = pair.split("=", 1)
        try:
            out[key] = json.loads(value)
        except json.JSONDecodeError:
            out[key] = value
    return out
