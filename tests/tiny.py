"""The tests' own tiny configurations and model folders.

Two Llama 3 configurations that differ in every size and option, written as the plain
``config.json`` dicts a model folder holds, and a folder writer that uses nothing of
the framework (torch's generator and the safetensors package).
"""

import json
import os

import torch

TINY_A = {
    "architectures": ["LlamaForCausalLM"],
    "vocab_size": 256,
    "hidden_size": 64,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "intermediate_size": 192,
    "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0,
    "max_position_embeddings": 128,
    "tie_word_embeddings": False,
}

TINY_B = {
    "architectures": ["LlamaForCausalLM"],
    "vocab_size": 512,
    "hidden_size": 128,
    "num_hidden_layers": 3,
    "num_attention_heads": 4,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "intermediate_size": 352,
    "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 64,
    },
    "max_position_embeddings": 256,
    "tie_word_embeddings": True,
}

# sizes that are no power of two anywhere: 3 query heads per kv head, head size 48,
# width 120 != heads * head size, vocabulary 331
TINY_C = {
    "architectures": ["LlamaForCausalLM"],
    "vocab_size": 331,
    "hidden_size": 120,
    "num_hidden_layers": 2,
    "num_attention_heads": 6,
    "num_key_value_heads": 2,
    "head_dim": 48,
    "intermediate_size": 200,
    "rms_norm_eps": 3e-6,
    "rope_theta": 25000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 4.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 2.0,
        "original_max_position_embeddings": 32,
    },
    "max_position_embeddings": 512,
    "tie_word_embeddings": False,
}


def tensor_shapes(cfg: dict) -> dict:
    d, f, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    h, k = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or d // h
    shapes = {"model.embed_tokens.weight": (v, d)}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        shapes[p + "input_layernorm.weight"] = (d,)
        shapes[p + "self_attn.q_proj.weight"] = (h * hd, d)
        shapes[p + "self_attn.k_proj.weight"] = (k * hd, d)
        shapes[p + "self_attn.v_proj.weight"] = (k * hd, d)
        shapes[p + "self_attn.o_proj.weight"] = (d, h * hd)
        shapes[p + "post_attention_layernorm.weight"] = (d,)
        shapes[p + "mlp.gate_proj.weight"] = (f, d)
        shapes[p + "mlp.up_proj.weight"] = (f, d)
        shapes[p + "mlp.down_proj.weight"] = (d, f)
    shapes["model.norm.weight"] = (d,)
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (v, d)
    return shapes


def random_weights(cfg: dict, seed: int, std: float = 0.02, norm_jitter: float = 0.1) -> dict:
    """N(0, std) matrices; norm weights 1 + a little noise so that a norm weight in
    the wrong place would show."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 1:
            out[name] = 1.0 + norm_jitter * torch.randn(shape, generator=gen)
        else:
            out[name] = std * torch.randn(shape, generator=gen)
    return out


def write_model_folder(folder: str, cfg: dict, weights: dict, dtype=torch.float32) -> str:
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def random_tokens(cfg: dict, n: int, seed: int) -> list:
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist()
