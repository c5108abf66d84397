import json
import os

import pytest
import torch

import tiny
from halite_amd.config import parse_config
from halite_amd.parts import Decoder
from halite_amd.weights import (
    ModelFiles,
    SafetensorsError,
    SafetensorsFile,
    WeightError,
    load_weights,
    save_file,
    write_random_model,
)


def _model(raw, dtype=torch.float32):
    arch, cfg = parse_config(raw)
    return arch, cfg, Decoder(arch.to_spec(cfg), dtype, "cpu")


def test_safetensors_round_trip_with_the_package(tmp_path):
    from safetensors.torch import load_file, save_file as pkg_save

    t = {
        "a": torch.randn(3, 5),
        "b": torch.randn(7).to(torch.bfloat16),
        "c": torch.arange(6, dtype=torch.int32).view(2, 3),
        "e": torch.empty(0, 4),
    }
    save_file(t, str(tmp_path / "ours.safetensors"))
    back = load_file(str(tmp_path / "ours.safetensors"))
    pkg_save(t, str(tmp_path / "theirs.safetensors"))
    f = SafetensorsFile(str(tmp_path / "theirs.safetensors"))
    for k in t:
        assert torch.equal(back[k], t[k]) and torch.equal(f.tensor(k), t[k])
    f.close()
    (tmp_path / "bad.safetensors").write_bytes(b"\xff" * 4)
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(tmp_path / "bad.safetensors"))
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        ModelFiles(str(tmp_path / "nowhere"))


@pytest.mark.parametrize("raw", [tiny.TINY_A, tiny.TINY_B])
def test_load_by_name(tmp_path, raw):
    arch, cfg, model = _model(raw)
    w = tiny.random_weights(raw, 3)
    tiny.write_model_folder(str(tmp_path), raw, w)
    load_weights(model, arch.weight_map(cfg), str(tmp_path))
    att = model.layers["1"].mixer
    nq = cfg.num_attention_heads * cfg.head_dim
    nk = cfg.num_key_value_heads * cfg.head_dim
    assert torch.equal(att.w_qkv[:nq], w["model.layers.1.self_attn.q_proj.weight"])
    assert torch.equal(att.w_qkv[nq : nq + nk], w["model.layers.1.self_attn.k_proj.weight"])
    assert torch.equal(att.w_qkv[nq + nk :], w["model.layers.1.self_attn.v_proj.weight"])
    ff = model.layers["0"].ff
    f = cfg.intermediate_size
    assert torch.equal(ff.w_gate_up[:f], w["model.layers.0.mlp.gate_proj.weight"])
    assert torch.equal(ff.w_gate_up[f:], w["model.layers.0.mlp.up_proj.weight"])
    assert torch.equal(model.final_norm.weight, w["model.norm.weight"])
    if cfg.tie_word_embeddings:
        assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()
    else:
        assert torch.equal(model.head.weight, w["lm_head.weight"])


def test_one_error_lists_everything(tmp_path):
    raw = tiny.TINY_A
    arch, cfg, model = _model(raw)
    w = tiny.random_weights(raw, 3)
    del w["model.layers.1.mlp.up_proj.weight"], w["model.norm.weight"]
    w["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    w["model.layers.7.extra.weight"] = torch.zeros(2)
    w["stray"] = torch.zeros(1)
    tiny.write_model_folder(str(tmp_path), raw, w)
    with pytest.raises(WeightError) as e:
        load_weights(model, arch.weight_map(cfg), str(tmp_path))
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert sorted(err.unexpected) == ["model.layers.7.extra.weight", "stray"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (16, 64))]
    text = str(err)
    for s in ("missing tensors (2)", "unexpected tensors (2)", "wrong shape", "[16, 64]", "[32, 64]", "stray"):
        assert s in text


def test_integer_and_unsupported_types(tmp_path):
    raw = tiny.TINY_A
    arch, cfg, model = _model(raw)
    w = tiny.random_weights(raw, 3)
    w["model.norm.weight"] = torch.ones(64, dtype=torch.int64)
    tiny_dir = str(tmp_path)
    from safetensors.torch import save_file as pkg_save

    os.makedirs(tiny_dir, exist_ok=True)
    with open(os.path.join(tiny_dir, "config.json"), "w") as f:
        json.dump(raw, f)
    pkg_save(w, os.path.join(tiny_dir, "model.safetensors"))
    with pytest.raises(WeightError, match="unsupported element type: model.norm.weight is I64"):
        load_weights(model, arch.weight_map(cfg), tiny_dir)


def test_element_types(tmp_path):
    raw = tiny.TINY_A
    w = tiny.random_weights(raw, 3)
    # stored in bfloat16, except one norm in 32-bit
    mixed = {k: v.to(torch.bfloat16) for k, v in w.items()}
    mixed["model.layers.0.input_layernorm.weight"] = w["model.layers.0.input_layernorm.weight"]
    from safetensors.torch import save_file as pkg_save

    (tmp_path / "config.json").write_text(json.dumps(raw))
    pkg_save(mixed, str(tmp_path / "model.safetensors"))
    arch, cfg, model = _model(raw, torch.bfloat16)
    load_weights(model, arch.weight_map(cfg), str(tmp_path))
    assert model.layers["0"].mixer.w_qkv.dtype == torch.bfloat16
    assert model.layers["0"].mixer_norm.weight.dtype == torch.float32  # a 32-bit tensor stays 32-bit
    assert model.layers["1"].mixer_norm.weight.dtype == torch.bfloat16
    arch, cfg, model = _model(raw, torch.float32)
    load_weights(model, arch.weight_map(cfg), str(tmp_path))
    assert model.layers["0"].mixer.w_qkv.dtype == torch.float32  # the 32-bit mode widens all
    assert torch.equal(model.embedding.weight, mixed["model.embed_tokens.weight"].float())


def test_tied_folder_may_carry_the_head(tmp_path):
    raw = tiny.TINY_B
    arch, cfg, model = _model(raw)
    w = tiny.random_weights(raw, 3)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    tiny.write_model_folder(str(tmp_path), raw, w)
    load_weights(model, arch.weight_map(cfg), str(tmp_path))
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()


@pytest.mark.parametrize("raw", [tiny.TINY_A, tiny.TINY_B])
def test_random_mode_writes_a_loadable_folder(tmp_path, raw):
    arch, cfg = parse_config(raw)
    a, b, c = (str(tmp_path / n) for n in "abc")
    write_random_model(a, cfg, seed=5, dtype="float32")
    write_random_model(b, cfg, seed=5, dtype="float32")
    write_random_model(c, cfg, seed=6, dtype="bfloat16")
    fa, fb, fc = ModelFiles(a), ModelFiles(b), ModelFiles(c)
    assert sorted(fa.names()) == sorted(tiny.tensor_shapes(raw))
    for name, shape in tiny.tensor_shapes(raw).items():
        ta = fa.tensor(name)
        assert tuple(ta.shape) == shape
        assert torch.equal(ta, fb.tensor(name))  # the seed decides
        if len(shape) == 1:
            assert torch.equal(ta, torch.ones(shape))
        else:
            assert not torch.equal(ta, fc.tensor(name).float())
            assert abs(float(ta.std()) - 0.02) < 0.004 and abs(float(ta.mean())) < 0.003
        assert fc.dtype_of(name) == "BF16"
    assert json.load(open(os.path.join(a, "config.json")))["rope_theta"] == raw["rope_theta"]
    _, cfg2, model = _model(json.load(open(os.path.join(a, "config.json"))))
    load_weights(model, arch.weight_map(cfg2), a)
    assert torch.equal(model.embedding.weight, fa.tensor("model.embed_tokens.weight"))
    for f in (fa, fb, fc):
        f.close()


def _two_shards(folder, raw, w, drop_from_shard=None, second_in=""):
    """The folder's tensors in two files and an index, as large models are stored."""
    from safetensors.torch import save_file as pkg_save

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f)
    names = list(w)
    first = {n: w[n].contiguous() for n in names[::2]}
    second = {n: w[n].contiguous() for n in names[1::2]}
    second_name = os.path.join(second_in, "model-00002-of-00002.safetensors")  # (an index may name a subfolder)
    os.makedirs(os.path.join(folder, second_in), exist_ok=True)
    index = {"metadata": {}, "weight_map": {**{n: "model-00001-of-00002.safetensors" for n in first},
                                            **{n: second_name for n in second}}}
    if drop_from_shard is not None:
        first.pop(drop_from_shard, None), second.pop(drop_from_shard, None)
    pkg_save(first, os.path.join(folder, "model-00001-of-00002.safetensors"))
    pkg_save(second, os.path.join(folder, second_name))
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f)


def test_a_folder_of_shards_loads_like_the_single_file(tmp_path):
    raw = tiny.TINY_A
    w = tiny.random_weights(raw, 4)
    one, two = str(tmp_path / "one"), str(tmp_path / "two")
    tiny.write_model_folder(one, raw, w)
    _two_shards(two, raw, w)
    arch, cfg, a = _model(raw)
    _, _, b = _model(raw)
    load_weights(a, arch.weight_map(cfg), one)
    load_weights(b, arch.weight_map(cfg), two)
    assert [s.path for s in a.param_slots()] == [s.path for s in b.param_slots()]
    for pa, pb in zip(a.named_parts().values(), b.named_parts().values()):
        for name in pa.param_decls():
            ta, tb = (getattr(p, name.replace(".", "_"), None) for p in (pa, pb))
            if ta is not None:
                assert torch.equal(ta, tb)
    assert torch.equal(a.layers["1"].mixer.w_qkv, b.layers["1"].mixer.w_qkv)
    assert torch.equal(a.layers["0"].parts()["ff"].w_gate_up, b.layers["0"].parts()["ff"].w_gate_up)
    assert torch.equal(a.head.weight, w["lm_head.weight"])


def test_a_missing_shard_and_a_tensor_missing_from_its_shard_are_named(tmp_path):
    raw = tiny.TINY_A
    w = tiny.random_weights(raw, 4)
    arch, cfg, model = _model(raw)
    gone = str(tmp_path / "gone")
    _two_shards(gone, raw, w)
    os.remove(os.path.join(gone, "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightError, match="missing shard file model-00002-of-00002.safetensors"):
        load_weights(model, arch.weight_map(cfg), gone)
    lacks = str(tmp_path / "lacks")
    _two_shards(lacks, raw, w, drop_from_shard="model.layers.1.mlp.up_proj.weight")
    with pytest.raises(WeightError) as e:
        load_weights(model, arch.weight_map(cfg), lacks)
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight"]
    assert "the index lists model.layers.1.mlp.up_proj.weight in model-0000" in str(e.value)
    with pytest.raises(WeightError, match="no model.safetensors and no model.safetensors.index.json"):
        load_weights(model, arch.weight_map(cfg), str(tmp_path / "nothing"))
    # a shard that the index names with a subfolder: found, and named so where it lacks a tensor
    deep = str(tmp_path / "deep")
    _two_shards(deep, raw, w, second_in="part2")
    load_weights(model, arch.weight_map(cfg), deep)
    assert torch.equal(model.head.weight, w["lm_head.weight"])
    deep_lacks = str(tmp_path / "deep_lacks")
    _two_shards(deep_lacks, raw, w, drop_from_shard=list(w)[1], second_in="part2")
    with pytest.raises(WeightError) as e:
        load_weights(model, arch.weight_map(cfg), deep_lacks)
    assert f"the index lists {list(w)[1]} in part2/model-00002" in str(e.value)
