"""A plain, slow Llama 3 decoder written from the reference's formulas.

Whole sequences, no cache, one function for each part, float32 on the CPU.  It
shares no code with ``halite_amd``: it reads ``config.json`` as a plain dict and
the weights as a plain ``{name: tensor}`` dict with the names a
``LlamaForCausalLM`` folder uses.  Citations are paths below the reference
checkout's root.
"""

from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------
# position encoding
# --------------------------------------------------------------------------


def inverse_frequencies(head_dim: int, theta: float) -> torch.Tensor:
    """``1 / theta^(2j/D)`` for ``j = 0 .. D/2-1`` in float32.

    src/halite/transformers/position.py:129-138
    """
    exponent = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    return 1 / (theta**exponent)


def llama3_scaled_frequencies(
    inv_freq: torch.Tensor,
    factor: float,
    low_freq_factor: float,
    high_freq_factor: float,
    original_context_len: int,
) -> torch.Tensor:
    """Llama 3 frequency scaling: long wavelengths are divided by ``factor``,
    short ones are kept, the band between is blended.

    src/halite/transformers/position.py:264-284
    """
    low_freq_wavelen = original_context_len / low_freq_factor
    high_freq_wavelen = original_context_len / high_freq_factor
    out = []
    for freq in inv_freq.tolist():
        freq = torch.tensor(freq, dtype=torch.float32)
        wavelen = 2 * math.pi / freq
        if wavelen > low_freq_wavelen:
            scaled = freq / factor
        else:
            scaled = freq
        if not (wavelen < high_freq_wavelen) and not (wavelen > low_freq_wavelen):
            smooth = (original_context_len / wavelen - low_freq_factor) / (
                high_freq_factor - low_freq_factor
            )
            scaled = (1 - smooth) * scaled / factor + smooth * scaled
        out.append(scaled)
    return torch.stack(out).to(torch.float32)


def rotation_table(positions: torch.Tensor, inv_freq: torch.Tensor):
    """``cos`` and ``sin`` of ``position * inv_freq[j]``, float32, ``[n, D/2]``.

    src/halite/transformers/position.py:140-167 (``torch.outer`` of float32
    positions and frequencies)
    """
    angles = torch.outer(positions.to(torch.float32), inv_freq)
    return angles.cos(), angles.sin()


def rotate_half_split(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor):
    """Pairs are ``(x[j], x[j + D/2])``: ``x*cos + rotate_half(x)*sin``.

    ``x`` is ``[n, heads, D]``; ``cos``/``sin`` are ``[n, D/2]``.
    src/halite/transformers/position.py:287-291, 346-365
    """
    half = x.shape[-1] // 2
    cos = torch.cat((cos, cos), -1).unsqueeze(1)
    sin = torch.cat((sin, sin), -1).unsqueeze(1)
    rotated = torch.cat((-x[..., half:], x[..., :half]), -1)
    return x * cos + rotated * sin


def rotate_interleaved(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor):
    """Pairs are the adjacent elements ``(x[2j], x[2j+1])``, multiplied as a
    complex number by ``cos + i sin``.

    src/halite/transformers/position.py:294-300
    """
    pairs = x.float().reshape(*x.shape[:-1], -1, 2)
    a, b = pairs[..., 0], pairs[..., 1]
    cos = cos.unsqueeze(1)
    sin = sin.unsqueeze(1)
    out = torch.stack((a * cos - b * sin, a * sin + b * cos), -1)
    return out.flatten(-2).type_as(x)


# --------------------------------------------------------------------------
# norm, feed-forward, embedding, head
# --------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, round_to=None) -> torch.Tensor:
    """``weight * (x32 * rsqrt(mean(x32^2) + eps)).type_as(x)``.

    With ``round_to`` the model's element type is that one: the normalised row is rounded to
    it before the weight multiplies it (the ``type_as``), and so is the product.

    src/halite/nn/normalization.py:43-57
    """
    x32 = x.to(torch.float32)
    normed = x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)
    if round_to is not None:
        return (weight * normed.to(round_to).float()).to(round_to).float()
    return weight * normed.type_as(x)


def gated_feed_forward(x, w_gate, w_up, w_down):
    """``down(up(x) * silu(gate(x)))``, no biases.

    src/halite/transformers/feedforward.py:204-212
    """
    gate = x @ w_gate.T
    up = x @ w_up.T
    return (up * (gate * torch.sigmoid(gate))) @ w_down.T


def embed(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """Row lookup, no multiplier.  src/halite/transformers/embedding.py:36-44"""
    return table[ids]


def output_head(hidden: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``hidden @ W^T`` in float32.
    src/halite/transformers/infer/postprocessor.py:45-57"""
    return (hidden @ weight.T).float()


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------


def causal_attention(q, k, v, window: int | None = None) -> torch.Tensor:
    """Softmax attention of a whole sequence.

    ``q`` is ``[n, H, D]``, ``k`` and ``v`` are ``[n, K, D]``; query head ``h``
    reads key/value head ``h // (H/K)``; the scale is ``1/sqrt(D)``; key ``j``
    is visible to query ``i`` iff ``j <= i`` (and ``j > i - window`` if a
    window is given); scores and softmax are float32.

    src/halite/transformers/attention.py:416-418 (scale), 647-714 (baddbmm,
    masked_fill, float32 softmax, ``attn @ value``), 600-609 (grouped heads)
    """
    n, n_heads, head_dim = q.shape
    group = n_heads // k.shape[1]
    scale = 1 / head_dim**0.5
    out = torch.empty_like(q)
    rows = torch.arange(n).unsqueeze(1)
    cols = torch.arange(n).unsqueeze(0)
    hidden = cols > rows
    if window is not None:
        hidden = hidden | (cols <= rows - window)
    for h in range(n_heads):
        g = h // group
        score = (q[:, h, :] @ k[:, g, :].T).float() * scale
        score = score.masked_fill(hidden, float("-inf"))
        prob = torch.softmax(score, -1, dtype=torch.float32).to(v.dtype)
        out[:, h, :] = prob @ v[:, g, :]
    return out


# --------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------


def read_model_folder(folder: str):
    """``config.json`` as a dict and ``model.safetensors`` as float32 tensors."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    weights = load_file(os.path.join(folder, "model.safetensors"))
    return config, {k: v.to(torch.float32) for k, v in weights.items()}


def rope_frequencies_of(config: dict) -> torch.Tensor:
    head_dim = config.get("head_dim") or (
        config["hidden_size"] // config["num_attention_heads"]
    )
    inv_freq = inverse_frequencies(head_dim, config.get("rope_theta", 10000.0))
    scaling = config.get("rope_scaling")
    if scaling is not None:
        kind = scaling.get("rope_type", scaling.get("type"))
        assert kind == "llama3", kind
        inv_freq = llama3_scaled_frequencies(
            inv_freq,
            scaling["factor"],
            scaling["low_freq_factor"],
            scaling["high_freq_factor"],
            scaling["original_max_position_embeddings"],
        )
    return inv_freq


def forward(config: dict, weights: dict, ids, position_offset: int = 0, round_to=None) -> torch.Tensor:
    """Logits ``[n, vocab]`` (float32) of one whole token sequence.

    The order in a layer is norm, q/k/v, rotation, attention, out, add, norm,
    gate/up, silu*mul, down, add.

    ``round_to`` (``torch.bfloat16``): a model whose element type is that one, emulated in
    float32: the result of every product, the rotated queries and keys, the attention's
    output, the activation and the norms' results are rounded to it; the norms' statistics,
    the rotation, the softmax and the residual sum stay float32 (the parts that are 32-bit
    whatever the model's type: src/halite/nn/normalization.py:43-57,
    src/halite/transformers/position.py:294-300, src/halite/transformers/attention.py:708).
    The arithmetic inside a product stays float32.  It says how far a model of that type may
    lie from 32-bit arithmetic through the number format alone.
    src/halite/transformers/block.py:56-74 (``x + module(pre_norm(x))``),
    src/halite/transformers/infer/attention.py:157-172,
    src/halite/transformers/infer/transformer.py:82-114
    """
    ids = torch.as_tensor(ids, dtype=torch.long)
    n = ids.shape[0]
    n_heads = config["num_attention_heads"]
    n_kv = config.get("num_key_value_heads") or n_heads
    head_dim = config.get("head_dim") or config["hidden_size"] // n_heads
    eps = config["rms_norm_eps"]
    interleaved = config.get("rope_interleaved", False)
    rotate = rotate_interleaved if interleaved else rotate_half_split

    cos, sin = rotation_table(
        torch.arange(n) + position_offset, rope_frequencies_of(config)
    )
    def r(t):
        return t if round_to is None else t.to(round_to).float()

    h = embed(ids, weights["model.embed_tokens.weight"])
    for i in range(config["num_hidden_layers"]):
        p = f"model.layers.{i}."
        x = rms_norm(h, weights[p + "input_layernorm.weight"], eps, round_to)
        q = r(x @ weights[p + "self_attn.q_proj.weight"].T).view(n, n_heads, head_dim)
        k = r(x @ weights[p + "self_attn.k_proj.weight"].T).view(n, n_kv, head_dim)
        v = r(x @ weights[p + "self_attn.v_proj.weight"].T).view(n, n_kv, head_dim)
        q = r(rotate(q, cos, sin))
        k = r(rotate(k, cos, sin))
        a = r(causal_attention(q, k, v)).reshape(n, n_heads * head_dim)
        h = h + r(a @ weights[p + "self_attn.o_proj.weight"].T)
        x = rms_norm(h, weights[p + "post_attention_layernorm.weight"], eps, round_to)
        if round_to is None:
            f = gated_feed_forward(
                x,
                weights[p + "mlp.gate_proj.weight"],
                weights[p + "mlp.up_proj.weight"],
                weights[p + "mlp.down_proj.weight"],
            )
        else:  # the same formula with the activation and the result rounded
            gate = x @ weights[p + "mlp.gate_proj.weight"].T
            up = x @ weights[p + "mlp.up_proj.weight"].T
            f = r(r(up * (gate * torch.sigmoid(gate))) @ weights[p + "mlp.down_proj.weight"].T)
        h = h + f
    h = rms_norm(h, weights["model.norm.weight"], eps, round_to)
    if config.get("tie_word_embeddings", False):
        head = weights["model.embed_tokens.weight"]
    else:
        head = weights["lm_head.weight"]
    return output_head(h, head)


# --------------------------------------------------------------------------
# sampling and generation
# --------------------------------------------------------------------------

_MASK64 = (1 << 64) - 1


def uniform_draw(seed: int, index: int) -> float:
    """The engine's counter-based uniform number for draw ``index`` of a
    request with ``seed``: a splitmix64 finaliser over the pair, top 24 bits.
    (The reference has no seed at all, src/halite/transformers/infer/engine/
    sampler.py:38-52 draws from the device generator; this stream is the
    engine's own, restated here from its definition.)
    """
    x = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xD1B54A32D192ED03) & _MASK64
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _MASK64
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _MASK64
    x ^= x >> 31
    return (x >> 40) / float(1 << 24)


def filtered_probabilities(
    logits: torch.Tensor,
    temperature: float,
    top_k: int = -1,
    top_p: float = 1.0,
    min_p: float = 0.0,
) -> torch.Tensor:
    """``softmax(logits / temperature)`` with the reference's filters.

    Without ``min_p`` the top-k and top-p filters are applied jointly (a token
    must pass both, both judged on the unfiltered distribution); with ``min_p``
    the order is top-k renormalise, top-p renormalise, then ``p >= min_p *
    max(p)``.  src/halite/transformers/infer/engine/sampler.py:32-52
    """
    probs = torch.softmax(logits.double() / temperature, -1)
    order = torch.argsort(probs, descending=True, stable=True)
    sorted_p = probs[order]
    keep_sorted = torch.ones_like(sorted_p, dtype=torch.bool)
    if top_k is not None and 0 < top_k < probs.numel():
        # everything as likely as the k-th token stays (ties are kept)
        keep_sorted &= sorted_p >= sorted_p[top_k - 1]
    if min_p > 0:
        kept_mass = sorted_p[keep_sorted].sum()
    else:
        kept_mass = sorted_p.sum()
    if top_p < 1.0:
        mass_before = torch.cumsum(sorted_p, 0) - sorted_p
        # a token stays while the tokens strictly more likely than it hold
        # less than top_p of the mass
        first_of_tie = torch.searchsorted(-sorted_p, -sorted_p, right=False)
        keep_sorted &= mass_before[first_of_tie] < top_p * kept_mass
    if min_p > 0:
        keep_sorted &= sorted_p >= min_p * sorted_p[0]
    keep = torch.zeros_like(keep_sorted)
    keep[order] = keep_sorted
    out = torch.where(keep, probs, torch.zeros_like(probs))
    return out / out.sum()


def sample_token(logits: torch.Tensor, params: dict, draw_index: int):
    """Next token and its log-probability.

    Greedy is ``temperature == 0`` or ``top_k == 1``: the first index of the
    maximum.  Otherwise the token is the first whose cumulative probability
    (in index order) exceeds the uniform draw.  The log-probability is that of
    the temperature-scaled, unfiltered distribution.
    src/halite/transformers/infer/engine/sampler.py:28-58
    """
    temperature = params.get("temperature", 1.0)
    top_k = params.get("top_k", -1)
    if temperature == 0 or top_k == 1:
        token = int(torch.argmax(logits))
        logprob = float(torch.log_softmax(logits.double(), -1)[token])
        return token, logprob, None
    probs = filtered_probabilities(
        logits, temperature, top_k, params.get("top_p", 1.0), params.get("min_p", 0.0)
    )
    u = uniform_draw(params.get("seed", 0), draw_index)
    cdf = torch.cumsum(probs, 0)
    token = int(torch.searchsorted(cdf, torch.tensor(u, dtype=cdf.dtype), right=True))
    token = min(token, probs.numel() - 1)
    logprob = float(torch.log_softmax(logits.double() / temperature, -1)[token])
    # distance of the draw to the nearest edge of the chosen token's interval:
    # a test may skip a comparison that rounding alone could flip
    lo = float(cdf[token - 1]) if token > 0 else 0.0
    margin = min(u - lo, float(cdf[token]) - u)
    return token, logprob, margin


def generate(config, weights, prompt, params: dict):
    """Token-by-token generation by running the whole sequence again each time.

    Stops after ``max_new_tokens`` or at a stop token (the stop token is part of
    the output).  src/halite/transformers/infer/engine/batch.py:180-204
    """
    ids = list(prompt)
    out, logprobs, margins = [], [], []
    stop = set(params.get("stop_token_ids") or ())
    for step in range(params.get("max_new_tokens", 128)):
        logits = forward(config, weights, ids)[-1]
        token, logprob, margin = sample_token(logits, params, step)
        out.append(token)
        logprobs.append(logprob)
        margins.append(margin)
        ids.append(token)
        if token in stop and not params.get("ignore_eos", False):
            break
    return out, logprobs, margins
