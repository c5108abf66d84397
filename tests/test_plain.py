"""Pins of the plain implementation: what fixes each formula beside the reference's
text.  Each check is chosen so that a plausible mistake (a wrong sign or pairing, a
norm in the wrong place, a wrong head mapping) fails it.  The reference holds no test
vectors for generation (its ``test/`` scripts print text for a human), so library
special cases and invariants stand in for them."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
import tiny


def test_inverse_frequencies_closed_form():
    f = P.inverse_frequencies(16, 10000.0)
    want = torch.tensor([10000.0 ** (-2 * j / 16) for j in range(8)])
    assert torch.allclose(f, want, rtol=1e-6)
    assert f[0] == 1.0 and f.shape == (8,)


def test_llama3_scaling_bands():
    # tiny B: original context 64, factor 8, low 1, high 4: all three bands occur
    f = P.inverse_frequencies(32, 500000.0)
    g = P.llama3_scaled_frequencies(f, 8.0, 1.0, 4.0, 64)
    wl = 2 * math.pi / f
    high, low = wl < 64 / 4.0, wl > 64 / 1.0
    mid = ~high & ~low
    assert high.any() and low.any() and mid.any()
    assert torch.equal(g[high], f[high])  # short wavelengths untouched
    assert torch.allclose(g[low], f[low] / 8.0, rtol=1e-6)  # long ones divided
    assert ((g[mid] < f[mid]) & (g[mid] > f[mid] / 8.0)).all()  # between, strictly
    assert (g[:-1] > g[1:]).all()  # still decreasing: no jump at a band's edge
    # factor 1 is the identity
    assert torch.allclose(P.llama3_scaled_frequencies(f, 1.0, 1.0, 4.0, 64), f, rtol=1e-6)


def test_llama3_scaling_meets_both_bands_at_their_edges():
    # What fixes the blend beside the reference's text: the scaled frequency is a
    # continuous function of the frequency.  On a dense sweep over all three bands the
    # ratio scaled/unscaled is 1 where wavelengths are short, 1/factor where they are
    # long, rises from the one to the other in between and meets both at the edges.  A
    # blend with its two weights swapped jumps by the factor at each edge; one that is
    # linear in the wavelength instead of the frequency is off in the middle.
    orig, factor, lo, hi = 8192, 8.0, 1.0, 4.0
    f_low_edge, f_high_edge = 2 * math.pi * lo / orig, 2 * math.pi * hi / orig
    f = torch.logspace(math.log10(f_low_edge / 30), math.log10(f_high_edge * 30), 4001, dtype=torch.float64).float()
    ratio = (P.llama3_scaled_frequencies(f, factor, lo, hi, orig) / f).double()
    fd = f.double()
    short, long_ = fd > f_high_edge * 1.0001, fd < f_low_edge * 0.9999
    mid = (fd > f_low_edge * 1.0001) & (fd < f_high_edge * 0.9999)
    assert short.sum() > 500 and long_.sum() > 500 and mid.sum() > 500
    assert torch.allclose(ratio[short], torch.ones_like(ratio[short]), atol=1e-6)
    assert torch.allclose(ratio[long_], torch.full_like(ratio[long_], 1 / factor), atol=1e-6)
    assert (ratio[1:] >= ratio[:-1] - 1e-6).all()  # never falls as the frequency rises
    assert ((ratio[mid] > 1 / factor) & (ratio[mid] < 1)).all()
    step = (ratio[1:] - ratio[:-1]).abs().max()
    assert step < 5e-3, f"the ratio jumps by {step} between neighbours of a dense sweep"
    # half-way between the edges in frequency, the ratio is half-way between 1/factor and 1
    middle = torch.tensor([(f_low_edge + f_high_edge) / 2], dtype=torch.float32)
    got = float(P.llama3_scaled_frequencies(middle, factor, lo, hi, orig) / middle)
    assert abs(got - (1 / factor + 1) / 2) < 1e-5


def test_llama3_scaling_of_the_8b_head():
    # head size 128 at the 8B's constants: six frequencies fall between the bands, so a
    # blend with swapped weights is no longer decreasing along the head
    f = P.inverse_frequencies(128, 500000.0)
    g = P.llama3_scaled_frequencies(f, 8.0, 1.0, 4.0, 8192)
    wl = 2 * math.pi / f
    mid = ~(wl < 8192 / 4.0) & ~(wl > 8192 / 1.0)
    assert int(mid.sum()) == 6
    assert (g[:-1] > g[1:]).all()
    assert ((g[mid] < f[mid]) & (g[mid] > f[mid] / 8.0)).all()
    s = (8192 * f[mid].double() / (2 * math.pi) - 1.0) / 3.0  # position between the edges, in frequency
    assert torch.allclose(g[mid].double() / f[mid].double(), (1 - s) / 8.0 + s, rtol=1e-5)


def test_llama3_scaling_matches_two_where_form():
    # the reference's vectorised form (src/halite/transformers/position.py:264-284)
    f = P.inverse_frequencies(64, 500000.0)
    orig, factor, lo, hi = 8192, 8.0, 1.0, 4.0
    wl = 2 * math.pi / f
    a = torch.where(wl > orig / lo, f / factor, f)
    s = (orig / wl - lo) / (hi - lo)
    b = (1 - s) * a / factor + s * a
    want = torch.where(~(wl < orig / hi) & ~(wl > orig / lo), b, a)
    assert torch.allclose(P.llama3_scaled_frequencies(f, factor, lo, hi, orig), want, rtol=1e-6)


def _qk(n=7, heads=3, d=16, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, heads, d, generator=g), torch.randn(n, heads, d, generator=g)


@pytest.mark.parametrize("rotate", [P.rotate_half_split, P.rotate_interleaved])
def test_rotation_is_a_rotation(rotate):
    q, _ = _qk()
    f = P.inverse_frequencies(16, 10000.0)
    cos, sin = P.rotation_table(torch.arange(7), f)
    r = rotate(q, cos, sin)
    assert torch.allclose(r[0], q[0], atol=1e-6)  # position 0: identity
    assert torch.allclose(r.norm(dim=-1), q.norm(dim=-1), rtol=1e-5)  # norms kept
    assert not torch.allclose(r[3], q[3], atol=1e-3)


@pytest.mark.parametrize("rotate", [P.rotate_half_split, P.rotate_interleaved])
def test_rotation_scores_depend_on_distance_only(rotate):
    q, k = _qk()
    f = P.inverse_frequencies(16, 10000.0)
    scores = []
    for shift in (0, 5, 40):
        cos, sin = P.rotation_table(torch.arange(7) + shift, f)
        rq, rk = rotate(q, cos, sin), rotate(k, cos, sin)
        scores.append(torch.einsum("ihd,jhd->hij", rq, rk))
    assert torch.allclose(scores[0], scores[1], atol=1e-4)
    assert torch.allclose(scores[0], scores[2], atol=1e-4)


def test_rotation_sign_and_pairing():
    # one pair, angle pi/2: (1, 0) -> (0, 1); a flipped sign gives (0, -1)
    x = torch.zeros(1, 1, 4)
    x[0, 0, 0] = 1.0
    cos, sin = torch.zeros(1, 2), torch.zeros(1, 2)
    cos[0, 1] = 1.0
    sin[0, 0] = 1.0
    h = P.rotate_half_split(x, cos, sin)
    assert torch.allclose(h[0, 0], torch.tensor([0.0, 0.0, 1.0, 0.0]))  # partner of 0 is 2
    i = P.rotate_interleaved(x, cos, sin)
    assert torch.allclose(i[0, 0], torch.tensor([0.0, 1.0, 0.0, 0.0]))  # partner of 0 is 1


def test_two_pairings_agree_under_the_permutation():
    # the adjacent pairing on x equals the half-split pairing on x with its
    # dimensions reordered [0, 2, 4, ..., 1, 3, 5, ...]
    q, _ = _qk(d=16)
    f = P.inverse_frequencies(16, 10000.0)
    cos, sin = P.rotation_table(torch.arange(7) + 3, f)
    perm = torch.cat((torch.arange(0, 16, 2), torch.arange(1, 16, 2)))
    a = P.rotate_interleaved(q, cos, sin)[..., perm]
    b = P.rotate_half_split(q[..., perm], cos, sin)
    assert torch.allclose(a, b, atol=1e-6)


def test_complex_form_equals_the_interleaved_rotation():
    # src/halite/transformers/position.py:294-300 multiplies complex numbers
    q, _ = _qk()
    f = P.inverse_frequencies(16, 10000.0)
    ang = torch.outer(torch.arange(7).float(), f)
    cis = torch.polar(torch.ones_like(ang), ang).unsqueeze(1)
    want = torch.view_as_real(torch.view_as_complex(q.reshape(7, 3, 8, 2)) * cis).flatten(-2)
    assert torch.allclose(P.rotate_interleaved(q, ang.cos(), ang.sin()), want, atol=1e-6)


def test_rms_norm():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 24, generator=g) * 3
    w = torch.randn(24, generator=g)
    want = F.rms_norm(x, (24,), None, 1e-5) * w
    assert torch.allclose(P.rms_norm(x, w, 1e-5), want, atol=1e-6)
    # invariant to the scale of x (for a small eps); the mean is over the width
    assert torch.allclose(P.rms_norm(7 * x, w, 1e-12), P.rms_norm(x, w, 1e-12), atol=1e-5)
    unit = x / x.pow(2).mean(-1, keepdim=True).sqrt()
    assert torch.allclose(P.rms_norm(unit, torch.ones(24), 1e-12), unit, atol=1e-5)
    # eps is inside the root
    tiny_x = torch.full((1, 4), 1e-4)
    assert torch.allclose(P.rms_norm(tiny_x, torch.ones(4), 1.0), tiny_x / math.sqrt(1e-8 + 1.0), rtol=1e-5)


def test_gated_feed_forward():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(4, 8, generator=g)
    wg, wu, wd = (torch.randn(s, generator=g) for s in ((12, 8), (12, 8), (8, 12)))
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(P.gated_feed_forward(x, wg, wu, wd), want, atol=1e-5)
    # gate and up are not interchangeable
    assert not torch.allclose(P.gated_feed_forward(x, wu, wg, wd), want, atol=1e-3)


@pytest.mark.parametrize("heads,kv", [(4, 4), (4, 2), (6, 1), (6, 2)])
def test_attention_reduces_to_sdpa(heads, kv):
    g = torch.Generator().manual_seed(3)
    n, d = 9, 8
    q = torch.randn(n, heads, d, generator=g)
    k = torch.randn(n, kv, d, generator=g)
    v = torch.randn(n, kv, d, generator=g)
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], is_causal=True, enable_gqa=True
    )[0].transpose(0, 1)
    assert torch.allclose(P.causal_attention(q, k, v), want, atol=1e-5)


def test_attention_special_cases():
    g = torch.Generator().manual_seed(4)
    q = torch.randn(6, 4, 8, generator=g)
    k = torch.randn(6, 2, 8, generator=g)
    v = torch.randn(6, 2, 8, generator=g)
    out = P.causal_attention(q, k, v)
    # the first token sees itself only: its output is its value, per group
    assert torch.allclose(out[0, 0], v[0, 0], atol=1e-6) and torch.allclose(out[0, 3], v[0, 1], atol=1e-6)
    # later keys never change an earlier row
    k2, v2 = k.clone(), v.clone()
    k2[4:] += 5.0
    v2[4:] -= 3.0
    assert torch.allclose(P.causal_attention(q, k2, v2)[:4], out[:4], atol=1e-6)
    # the same value everywhere comes out unchanged
    same = v[:1].expand(6, 2, 8)
    assert torch.allclose(P.causal_attention(q, k, same), same.repeat_interleave(2, 1), atol=1e-5)
    # a window of 1 sees only the token itself; a window beyond the length changes nothing
    assert torch.allclose(P.causal_attention(q, k, v, window=1), v.repeat_interleave(2, 1), atol=1e-6)
    assert torch.allclose(P.causal_attention(q, k, v, window=6), out, atol=1e-6)
    assert not torch.allclose(P.causal_attention(q, k, v, window=2), out, atol=1e-3)


def test_attention_scale_is_inverse_root_of_head_size():
    # one query against two keys: probabilities follow from the scaled scores
    q = torch.tensor([[[0.0] * 16], [[2.0] + [0.0] * 15]])
    k = torch.tensor([[[4.0] + [0.0] * 15], [[0.0] * 16]])
    v = torch.tensor([[[1.0] + [0.0] * 15], [[0.0] * 16]])
    out = P.causal_attention(q, k, v)
    p = torch.softmax(torch.tensor([2.0 * 4.0 / 4.0, 0.0]), 0)[0]
    assert torch.allclose(out[1, 0, 0], p, atol=1e-6)


def test_model_shift_invariance_and_causality():
    cfg = tiny.TINY_B
    w = tiny.random_weights(cfg, 7, std=0.05)
    ids = tiny.random_tokens(cfg, 12, 1)
    a = P.forward(cfg, w, ids)
    b = P.forward(cfg, w, ids, position_offset=17)
    assert torch.allclose(a, b, atol=2e-5)  # only distances count
    c = P.forward(cfg, w, ids[:8])
    assert torch.allclose(a[:8], c, atol=1e-5)  # a prefix's logits do not see the rest
    # tied head: the logits are hidden @ embedding^T.  Another table handed in as a head is
    # not looked at, and the logits follow the embedding table's rows
    decoy = dict(w)
    decoy["lm_head.weight"] = torch.randn_like(w["model.embed_tokens.weight"])
    assert torch.equal(P.forward(cfg, decoy, ids), a)
    swapped = dict(w)
    table = w["model.embed_tokens.weight"].clone()
    unused = [t for t in range(cfg["vocab_size"]) if t not in ids][:2]
    table[unused] = table[unused[::-1]]  # two rows that no token of the input reads
    swapped["model.embed_tokens.weight"] = table
    d = P.forward(cfg, swapped, ids)
    assert torch.equal(d[:, unused], a[:, unused[::-1]]) and not torch.equal(d[:, unused], a[:, unused])
    # the same weights read as untied: the other table is the head then
    assert not torch.allclose(P.forward(dict(cfg, tie_word_embeddings=False), decoy, ids), a, atol=1e-3)


def library_model(cfg, w, ids):
    """The whole model once more, from library routines alone and in the reference's own
    formulation where it has one: ``F.embedding``, ``F.rms_norm``, ``F.linear``, the rotation
    as a product of complex numbers (src/halite/transformers/position.py:140-167, 294-300),
    ``F.scaled_dot_product_attention`` with ``is_causal`` and ``enable_gqa``
    (src/halite/transformers/attention.py:600-609), ``F.silu``; a sub-block is
    ``input + module(pre_norm(input))`` (src/halite/transformers/block.py:56-74), the last
    norm and the head follow the last block (src/halite/transformers/infer/transformer.py:
    105-112).  For configurations with ``rope_interleaved``."""
    n = len(ids)
    H, K = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    D = cfg.get("head_dim") or cfg["hidden_size"] // H
    eps, width = cfg["rms_norm_eps"], (cfg["hidden_size"],)
    freq = 1.0 / cfg["rope_theta"] ** (torch.arange(0, D, 2, dtype=torch.float32) / D)
    sc = cfg.get("rope_scaling")
    if sc is not None:  # the two-where form of src/halite/transformers/position.py:264-284
        orig, factor = sc["original_max_position_embeddings"], sc["factor"]
        lo, hi = sc["low_freq_factor"], sc["high_freq_factor"]
        wl = 2 * math.pi / freq
        first = torch.where(wl > orig / lo, freq / factor, freq)
        smooth = (orig / wl - lo) / (hi - lo)
        freq = torch.where(~(wl < orig / hi) & ~(wl > orig / lo), (1 - smooth) * first / factor + smooth * first, first)
    ang = torch.outer(torch.arange(n, dtype=torch.float32), freq)
    cis = torch.polar(torch.ones_like(ang), ang).unsqueeze(1)

    def rotate(x):
        return torch.view_as_real(torch.view_as_complex(x.float().reshape(n, -1, D // 2, 2)) * cis).flatten(-2)

    h = F.embedding(torch.as_tensor(ids), w["model.embed_tokens.weight"])
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        x = F.rms_norm(h, width, w[p + "input_layernorm.weight"], eps)
        q = rotate(F.linear(x, w[p + "self_attn.q_proj.weight"]).view(n, H, D))
        k = rotate(F.linear(x, w[p + "self_attn.k_proj.weight"]).view(n, K, D))
        v = F.linear(x, w[p + "self_attn.v_proj.weight"]).view(n, K, D)
        a = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                           is_causal=True, enable_gqa=True)[0].transpose(0, 1).reshape(n, H * D)
        h = h + F.linear(a, w[p + "self_attn.o_proj.weight"])
        x = F.rms_norm(h, width, w[p + "post_attention_layernorm.weight"], eps)
        h = h + F.linear(F.silu(F.linear(x, w[p + "mlp.gate_proj.weight"])) * F.linear(x, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return F.linear(F.rms_norm(h, width, w["model.norm.weight"], eps), head)


def rows_for_half_split(cfg, w):
    """The same model stored for the half-split pairing: the rows of every head of the
    query and key matrices reordered [0, 2, 4, ..., 1, 3, 5, ...]."""
    D = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
    perm = torch.cat((torch.arange(0, D, 2), torch.arange(1, D, 2)))
    out = dict(w)
    for name, t in w.items():
        if name.endswith(("q_proj.weight", "k_proj.weight")):
            out[name] = t.view(-1, D, t.shape[1])[:, perm].reshape(t.shape)
    return out


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_model_against_library_routines(name):
    """Pins every formula and the order of a block at once: the plain implementation
    against a model made of library routines (an outside model library is not used as a
    yardstick here: model code of installed packages is no source for this repository).
    Then the half-split pairing, which model folders are stored for, against the adjacent
    one on the reordered rows."""
    cfg = dict({"A": tiny.TINY_A, "B": tiny.TINY_B, "C": tiny.TINY_C}[name], rope_interleaved=True)
    w = tiny.random_weights(cfg, 21, std=0.08)
    for n, seed in ((1, 1), (37, 2), (cfg["max_position_embeddings"] // 2, 3)):
        ids = tiny.random_tokens(cfg, n, seed)
        want = library_model(cfg, w, ids)
        got = P.forward(cfg, w, ids)
        assert float((got - want).abs().max()) <= 1e-5 * max(1.0, float(want.abs().max())), (name, n)
        half = P.forward(dict(cfg, rope_interleaved=False), rows_for_half_split(cfg, w), ids)
        assert float((half - want).abs().max()) <= 1e-5 * max(1.0, float(want.abs().max())), (name, n)
    # what the comparison would catch: a residual taken after the norm, a norm left out
    broken = dict(w)
    broken["model.norm.weight"] = torch.ones_like(w["model.norm.weight"])
    assert float((P.forward(cfg, broken, ids) - want).abs().max()) > 1e-3


def test_norm_weight_position_matters():
    cfg = tiny.TINY_A
    w = tiny.random_weights(cfg, 8, std=0.05)
    ids = tiny.random_tokens(cfg, 6, 2)
    a = P.forward(cfg, w, ids)
    w2 = dict(w)
    w2["model.layers.0.input_layernorm.weight"], w2["model.layers.0.post_attention_layernorm.weight"] = (
        w["model.layers.0.post_attention_layernorm.weight"],
        w["model.layers.0.input_layernorm.weight"],
    )
    assert not torch.allclose(a, P.forward(cfg, w2, ids), atol=1e-4)


def test_uniform_draw_is_a_uniform_stream():
    us = [P.uniform_draw(123, i) for i in range(4000)]
    assert all(0.0 <= u < 1.0 for u in us)
    assert abs(sum(us) / len(us) - 0.5) < 0.02
    assert len(set(us)) > 3990
    assert P.uniform_draw(123, 5) == P.uniform_draw(123, 5) != P.uniform_draw(124, 5)


def test_filters():
    logits = torch.log(torch.tensor([0.5, 0.2, 0.2, 0.06, 0.04]))
    p = P.filtered_probabilities(logits, 1.0)
    assert torch.allclose(p, torch.tensor([0.5, 0.2, 0.2, 0.06, 0.04], dtype=p.dtype), atol=1e-6)
    p = P.filtered_probabilities(logits, 1.0, top_k=2)  # the tie at 0.2 stays whole
    assert (p > 0).tolist() == [True, True, True, False, False]
    p = P.filtered_probabilities(logits, 1.0, top_p=0.6)
    assert (p > 0).tolist() == [True, True, True, False, False]
    p = P.filtered_probabilities(logits, 1.0, top_p=0.45)
    assert (p > 0).tolist() == [True, False, False, False, False]
    p = P.filtered_probabilities(logits, 1.0, min_p=0.2)  # p >= 0.2 * 0.5
    assert (p > 0).tolist() == [True, True, True, False, False]
    assert abs(float(p.sum()) - 1.0) < 1e-9
    hot = P.filtered_probabilities(logits, 0.05)
    assert hot[0] > 0.999  # temperature -> 0 approaches the maximum


def test_sample_token_greedy_and_draw():
    logits = torch.tensor([0.1, 2.0, 2.0, -1.0])
    tok, lp, _ = P.sample_token(logits, {"temperature": 0.0}, 0)
    assert tok == 1 and abs(lp - float(torch.log_softmax(logits.double(), -1)[1])) < 1e-9
    assert P.sample_token(logits, {"top_k": 1, "temperature": 0.7}, 0)[0] == 1
    counts = torch.zeros(4)
    for i in range(3000):
        counts[P.sample_token(logits, {"temperature": 1.0, "seed": 9}, i)[0]] += 1
    want = torch.softmax(logits, -1) * 3000
    assert ((counts - want).abs() < 4 * want.sqrt() + 5).all()


def test_rounding_mode_rounds_where_it_says():
    """``round_to`` emulates a model of that element type: float32 changes nothing, bfloat16
    moves the logits by about its precision per rounding, and what is rounded is what the
    docstring lists (a product's result: one layer's q, k, v are on the bfloat16 grid)."""
    cfg = tiny.TINY_C
    w = {k: v.to(torch.bfloat16).float() for k, v in tiny.random_weights(cfg, 5, std=0.06).items()}
    ids = tiny.random_tokens(cfg, 40, 3)
    exact = P.forward(cfg, w, ids)
    assert torch.equal(P.forward(cfg, w, ids, round_to=torch.float32), exact)
    rounded = P.forward(cfg, w, ids, round_to=torch.bfloat16)
    err = float((rounded - exact).abs().max()) / float(exact.abs().max())
    assert 1e-4 < err < 2e-2, err
    x = torch.randn(5, cfg["hidden_size"])
    weight = w["model.norm.weight"]
    y = P.rms_norm(x, weight, 1e-6, torch.bfloat16)
    assert torch.equal(y, y.to(torch.bfloat16).float())
    inner = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16).float()
    assert torch.equal(y, (weight * inner).to(torch.bfloat16).float())  # rounded before the weight, as type_as does
