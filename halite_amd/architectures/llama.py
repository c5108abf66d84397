"""Llama 3 as the reference defines it (configs/models/llama/llama3_2_3b.py:12-57 on
top of configs/models/transformer.py:201-311): token embedding, pre-norm blocks of
grouped-query attention with rotary positions and a SiLU-gated feed-forward, a final
RMSNorm and a bias-free head that may share the embedding's table.
"""

from __future__ import annotations

from ..config.model import LlamaConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import LayerRun, LayerSpec, ModelSpec, PartSpec


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    rope = dict(
        kind="rope",
        head_dim=cfg.head_dim,
        rotary_dim=cfg.head_dim,
        theta=cfg.rope_theta,
        interleaved=cfg.rope_interleaved,
        max_positions=cfg.max_position_embeddings,
    )
    if cfg.rope_scaling is not None:
        sc = cfg.rope_scaling  # "llama3" is the only type the configuration lets through
        rope["scaling"] = dict(
            kind="banded",
            factor=sc.factor,
            low_freq_factor=sc.low_freq_factor,
            high_freq_factor=sc.high_freq_factor,
            original_context_len=sc.original_max_position_embeddings,
        )
    norm = PartSpec(kind="rmsnorm", size=cfg.hidden_size, eps=cfg.rms_norm_eps)
    layer = LayerSpec(arrangement="pre_norm", parts=dict(
        mixer_norm=norm,
        mixer=PartSpec(
            kind="attention",
            hidden_size=cfg.hidden_size,
            n_heads=cfg.num_attention_heads,
            n_kv_heads=cfg.num_key_value_heads,
            head_dim=cfg.head_dim,
            # configs/models/transformer.py: normalize=True -> 1/sqrt(head_dim)
            # (src/halite/transformers/attention.py:416-418)
            scale=cfg.head_dim**-0.5,
            position="rope",
            window=None,
        ),
        ff_norm=norm,
        ff=PartSpec(
            kind="gated",
            hidden_size=cfg.hidden_size,
            intermediate_size=cfg.intermediate_size,
            activation=cfg.hidden_act,
        ),
    ))
    names = [str(i) for i in range(cfg.num_hidden_layers)]
    return ModelSpec(
        architecture="LlamaForCausalLM",
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec(kind="embedding", vocab_size=cfg.vocab_size, size=cfg.hidden_size),
        positions={"rope": PartSpec(**rope)},
        layers={name: layer for name in names},
        order=[LayerRun(layer=name) for name in names],
        final_norm=norm,
        head=PartSpec(
            kind="linear_head",
            vocab_size=cfg.vocab_size,
            size=cfg.hidden_size,
            tied=cfg.tie_word_embeddings,
        ),
    )


def llama_weight_map(cfg: LlamaConfig) -> dict[str, str | None]:
    """Tensor name in the folder -> parameter of a part.  The right-hand sides
    follow the reference's own keys (``q``, ``k``, ``v``, ``out``, ``linear_gate``,
    ``linear_proj``, ``linear_out``; configs/models/llama/checkpoint.py:94-158)."""
    table = {
        "model.embed_tokens.weight": "embedding.weight",
        "model.layers.#.input_layernorm.weight": "layers.#.mixer_norm.weight",
        "model.layers.#.self_attn.q_proj.weight": "layers.#.mixer.q.weight",
        "model.layers.#.self_attn.k_proj.weight": "layers.#.mixer.k.weight",
        "model.layers.#.self_attn.v_proj.weight": "layers.#.mixer.v.weight",
        "model.layers.#.self_attn.o_proj.weight": "layers.#.mixer.out.weight",
        "model.layers.#.post_attention_layernorm.weight": "layers.#.ff_norm.weight",
        "model.layers.#.mlp.gate_proj.weight": "layers.#.ff.linear_gate.weight",
        "model.layers.#.mlp.up_proj.weight": "layers.#.ff.linear_proj.weight",
        "model.layers.#.mlp.down_proj.weight": "layers.#.ff.linear_out.weight",
        "model.norm.weight": "final_norm.weight",
    }
    # a tied model's folder may still carry a copy of the table under the head's
    # name; None marks a name that is passed over if present
    table["lm_head.weight"] = None if cfg.tie_word_embeddings else "head.weight"
    return table


LLAMA = register_architecture(
    Architecture(
        name="LlamaForCausalLM",
        config_cls=LlamaConfig,
        to_spec=llama_spec,
        weight_map=llama_weight_map,
    )
)
