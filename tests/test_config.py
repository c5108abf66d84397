import json

import pytest

import tiny
from halite_amd.config import (
    ConfigError,
    LlamaConfig,
    ModelConfig,
    ModelSpec,
    ServerConfig,
    get_architecture,
    parse_config,
    parse_overrides,
    read_config,
)


def test_parses_both_tiny_configs():
    for raw in (tiny.TINY_A, tiny.TINY_B, tiny.TINY_C):
        arch, cfg = parse_config(raw)
        assert arch.name == "LlamaForCausalLM"
        assert isinstance(cfg, LlamaConfig)
        assert cfg.head_dim == raw["head_dim"] and cfg.rms_norm_eps == raw["rms_norm_eps"]
        assert cfg.rope_theta == raw["rope_theta"]
    _, b = parse_config(tiny.TINY_B)
    assert b.rope_scaling.factor == 8.0 and b.rope_scaling.original_max_position_embeddings == 64
    assert b.tie_word_embeddings is True


def test_defaults_that_have_a_meaning():
    raw = dict(tiny.TINY_A)
    del raw["num_key_value_heads"], raw["head_dim"]
    _, cfg = parse_config(raw)
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 16 and cfg.rope_scaling is None


def test_other_spellings_of_the_rotation_keys():
    # base and scaling arguments in one dict, as newer writers of such folders do
    raw = dict(tiny.TINY_B)
    merged = dict(raw.pop("rope_scaling"), rope_theta=raw.pop("rope_theta"))
    raw["rope_parameters"] = merged
    _, cfg = parse_config(raw)
    _, ref = parse_config(tiny.TINY_B)
    assert cfg.rope_theta == ref.rope_theta and cfg.rope_scaling == ref.rope_scaling
    # "default" names the unscaled frequencies
    raw = dict(tiny.TINY_A, rope_scaling={"rope_type": "default"})
    assert parse_config(raw)[1].rope_scaling is None
    raw = dict(tiny.TINY_A)
    raw["rope_parameters"] = {"rope_type": "default", "rope_theta": raw.pop("rope_theta")}
    cfg = parse_config(raw)[1]
    assert cfg.rope_scaling is None and cfg.rope_theta == tiny.TINY_A["rope_theta"]
    # and still no default for the base
    raw = dict(tiny.TINY_A)
    del raw["rope_theta"]
    raw["rope_parameters"] = {"rope_type": "default"}
    with pytest.raises(ConfigError, match="rope_theta"):
        parse_config(raw)


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "intermediate_size", "rms_norm_eps", "rope_theta", "max_position_embeddings"])
def test_no_size_has_a_default_in_code(key):
    raw = dict(tiny.TINY_A)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        parse_config(raw)


@pytest.mark.parametrize(
    "change,match",
    [
        ({"num_key_value_heads": 3}, "not a multiple"),
        ({"head_dim": 15}, "odd"),
        ({"attention_bias": True}, "bias"),
        ({"mlp_bias": True}, "bias"),
        ({"hidden_act": "gelu"}, "silu"),
        ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "llama3"),
        ({"rope_scaling": {"rope_type": "llama3", "factor": 2.0}}, "low_freq_factor"),
        ({"vocab_size": "256"}, "vocab_size"),
        ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ],
)
def test_validation_errors(change, match):
    with pytest.raises(ConfigError, match=match):
        parse_config({**tiny.TINY_A, **change})


def test_unknown_architecture_lists_known():
    with pytest.raises(ConfigError, match="LlamaForCausalLM"):
        parse_config({**tiny.TINY_A, "architectures": ["MambaForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        parse_config({k: v for k, v in tiny.TINY_A.items() if k != "architectures"})


def test_round_trip_through_json(tmp_path):
    _, cfg = parse_config(tiny.TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_json_dict()))
    _, again = read_config(str(tmp_path))
    assert again == cfg
    with pytest.raises(ConfigError, match="config.json"):
        read_config(str(tmp_path / "nothing"))


def test_spec_is_data():
    arch, cfg = parse_config(tiny.TINY_B)
    spec = arch.to_spec(cfg)
    assert [r.layer for r in spec.order] == ["0", "1", "2"]
    assert sorted(spec.layers["1"].parts) == ["ff", "ff_norm", "mixer", "mixer_norm"]
    att = spec.layers["1"].parts["mixer"]
    assert att.kind == "attention" and att.params()["n_kv_heads"] == 1 and att.params()["head_dim"] == 32
    assert abs(att.params()["scale"] - 32**-0.5) < 1e-12
    assert spec.positions["rope"].params()["scaling"]["factor"] == 8.0
    assert spec.head.params()["tied"] is True
    again = ModelSpec(**json.loads(spec.model_dump_json()))
    assert again == spec
    # the run order is validated as data too
    bad = spec.model_dump()
    bad["order"][1]["cache_from"] = 2
    with pytest.raises(ValueError, match="earlier run"):
        ModelSpec(**bad)
    bad = spec.model_dump()
    bad["order"][0]["layer"] = "nope"
    with pytest.raises(ValueError, match="unknown layer"):
        ModelSpec(**bad)


def test_a_layer_names_the_parts_its_arrangement_has():
    import torch

    from halite_amd.config.registry import ConfigError
    from halite_amd.parts import Decoder

    arch, cfg = parse_config(tiny.TINY_A)
    spec = arch.to_spec(cfg)
    Decoder(spec, torch.float32, "cpu")  # builds
    norm = spec.layers["0"].parts["ff_norm"]
    # a part that the arrangement does not have is refused, not dropped
    extra = spec.model_copy(deep=True)
    extra.layers["1"].parts["post_norm"] = norm
    with pytest.raises(ConfigError, match=r"no part named \['post_norm'\]"):
        Decoder(extra, torch.float32, "cpu")
    # and so is a layer that leaves one out
    short = spec.model_copy(deep=True)
    del short.layers["0"].parts["ff_norm"]
    with pytest.raises(ConfigError, match=r"leaves out \['ff_norm'\]"):
        Decoder(short, torch.float32, "cpu")
    other = spec.model_copy(deep=True)
    other.layers["0"].arrangement = "post_norm"
    with pytest.raises(ConfigError, match="unknown arrangement 'post_norm'; known: pre_norm"):
        Decoder(other, torch.float32, "cpu")
    # the keyword form and the dict form are the same description
    from halite_amd.config import LayerSpec

    parts = spec.layers["0"].parts
    assert LayerSpec(**parts) == LayerSpec(arrangement="pre_norm", parts=parts) == spec.layers["0"]


def test_weight_map_names():
    arch = get_architecture("LlamaForCausalLM")
    _, a = parse_config(tiny.TINY_A)
    _, b = parse_config(tiny.TINY_B)
    assert arch.weight_map(a)["lm_head.weight"] == "head.weight"
    assert arch.weight_map(b)["lm_head.weight"] is None
    assert arch.weight_map(a)["model.layers.#.mlp.up_proj.weight"] == "layers.#.ff.linear_proj.weight"


def test_engine_options_and_overrides():
    s = ServerConfig(**parse_overrides(["page_size=16", "max_tokens_per_forward=512", "use_cudagraph=true"]))
    assert s.page_size == 16 and s.max_tokens_per_forward == 512 and s.use_cudagraph is True
    assert s.max_prefill_tokens == 16384 and s.chunked_prefill_size == 8192  # the reference's defaults
    assert s.default_init_new_token_ratio == 0.7
    # the reference's way to list graph sizes (infer/types.py:77-80), its spelling included
    assert s.cudagraph_step == 16 and s.cudagraph_additonal_batch_size == ()
    s = ServerConfig(**parse_overrides(["cudagraph_step=8", "cudagraph_additonal_batch_size=[1, 2, 4]"]))
    assert s.cudagraph_step == 8 and s.cudagraph_additonal_batch_size == (1, 2, 4)
    with pytest.raises(ValueError):
        ServerConfig(cudagraph_step=0)
    with pytest.raises(ValueError):
        ServerConfig(page_size=0)
    with pytest.raises(ValueError):
        ServerConfig(no_such_option=1)
    with pytest.raises(ValueError):
        ModelConfig(dtype="float16")
    with pytest.raises(ValueError, match="key=value"):
        parse_overrides(["page_size"])
    # what the reference's callers tell its engine about the model (scripts/eval_task.py:148-154)
    # is taken and checked against the model; several GPUs are not
    from halite_amd.config.engine import check_stated_sizes

    stated = ModelConfig(n_heads=6, n_key_value_heads=2, head_dim=48, n_layers=3, context_len=256)
    check_stated_sizes(stated, 3, [(6, 2, 48)] * 3)
    check_stated_sizes(ModelConfig(), 5, [(4, 4, 16), (8, 2, 32)])  # nothing stated, nothing to check
    with pytest.raises(ValueError, match=r"n_layers=3 \(the model runs 4\).*head_dim=48 \(the model's layers have 32, 48\)"):
        check_stated_sizes(stated, 4, [(6, 2, 48), (6, 2, 32)])
    with pytest.raises(ValueError):
        ModelConfig(tp_size=2)
    with pytest.raises(ValueError):
        ModelConfig(distributed=True)


def test_command_line_takes_overrides_and_options_in_any_order():
    from halite_amd.cli.generate import parse_args, split_overrides

    args = parse_args(["--model", "DIR", "sampling.max_new_tokens=4", "--prompt-ids", "1,2,3",
                       "server.page_size=16", "--stats", "model.dtype=float32"])
    assert args.model == "DIR" and args.prompt_ids == ["1,2,3"] and args.stats
    over = split_overrides(args.opts)
    assert over == {"sampling": {"max_new_tokens": 4}, "server": {"page_size": 16}, "model": {"dtype": "float32"}}
    with pytest.raises(SystemExit):
        split_overrides(["foo=1"])


def test_an_architecture_must_bring_what_the_framework_reads_of_its_configuration():
    """``architectures`` is the one field that generic code reads of a configuration class;
    a class without it is refused when it is registered, not when a folder is written."""
    from pydantic import BaseModel

    from halite_amd.config.registry import ARCHITECTURES, Architecture, ConfigError, register_architecture

    class Nameless(BaseModel):
        width: int

    with pytest.raises(ConfigError, match="architectures"):
        register_architecture(Architecture("NamelessLM", Nameless, lambda c: None, lambda c: {}))
    assert "NamelessLM" not in ARCHITECTURES

    class Named(BaseModel):
        architectures: list[str]
        width: int

    try:
        assert register_architecture(Architecture("NamedLM", Named, lambda c: None, lambda c: {})).name == "NamedLM"
    finally:
        ARCHITECTURES.pop("NamedLM", None)
