"""The parts alone, and models put together from parts as data: a windowed layer, a
layer that runs twice, a layer that reads another layer's cache, and toy parts that are
defined here and registered without touching the framework: a mixer with state of its
own, a mixer whose pages hold something else than keys and values, a feed-forward that
routes tokens to experts, and another position encoding."""

from dataclasses import dataclass

import pytest
import torch
from pydantic import BaseModel

import plain_llama as P
import replay
import tiny
from halite_amd.config import LayerRun, LayerSpec, ModelConfig, ModelSpec, PartSpec, ServerConfig, parse_config
from halite_amd.engine.batch import Segment
from halite_amd.engine.runner import ModelRunner
from halite_amd.parts import MIXERS, BuildContext, Decoder, Mixer, PagedNeed, ParamDecl, StateNeed
from halite_amd.parts.base import FEED_FORWARDS, NORMS, POSITIONS, Arrangement, FeedForward, PositionEncoding, register_arrangement
from halite_amd.weights import fill_random

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 5e-5, "bfloat16": 2.5e-2}


def build(gpu, dtype):
    return BuildContext(dtype=DT[dtype], device=gpu, hidden_size=0)


def fill(part, dtype, seed=0, std=0.05):
    """Random tensors for one part, returned as float32 CPU copies by name."""
    decls = part.param_decls()
    views = part.allocate({n: DT[dtype] for n in decls})
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, d in decls.items():
        t = 1 + 0.1 * torch.randn(d.shape, generator=g) if d.init == "ones" else std * torch.randn(d.shape, generator=g)
        views[name].copy_(t)
        out[name] = views[name].float().cpu()
    part.finalize()
    return out


@pytest.mark.parametrize("raw", [tiny.TINY_A, tiny.TINY_B, tiny.TINY_C])
def test_rope_part(gpu, raw):
    arch, cfg = parse_config(raw)
    rope = POSITIONS.build(arch.to_spec(cfg).positions["rope"], build(gpu, "float32"))
    want = P.rope_frequencies_of(raw)
    assert torch.equal(rope.inv_freq, want)
    cos, sin = rope.tables(100)
    c, s = P.rotation_table(torch.arange(cos.shape[0]), want)
    assert torch.equal(cos.cpu(), c) and torch.equal(sin.cpu(), s)
    more = rope.tables(cfg.max_position_embeddings)[0]
    assert more.shape[0] >= cfg.max_position_embeddings and torch.equal(more[:100].cpu(), c[:100])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_and_feed_forward_parts(gpu, dtype):
    b = build(gpu, dtype)
    norm = NORMS.build(PartSpec(kind="rmsnorm", size=120, eps=1e-5), b)
    w = fill(norm, dtype, 1)["weight"]
    h = torch.randn(70, 120, generator=torch.Generator().manual_seed(2))
    got = norm.forward(h.to(gpu).clone())
    err = float((got.float().cpu() - P.rms_norm(h, w, 1e-5)).abs().max())
    assert err < (1e-5 if dtype == "float32" else 3e-2)

    ff = FEED_FORWARDS.build(PartSpec(kind="gated", hidden_size=120, intermediate_size=200, activation="silu"), b)
    ws = fill(ff, dtype, 3, std=0.1)
    for rows in (5, 64, 70):  # the fused small-batch kernel and the large-batch path
        x = torch.randn(rows, 120, generator=torch.Generator().manual_seed(rows)).to(DT[dtype])
        want = P.gated_feed_forward(x.float(), ws["linear_gate.weight"], ws["linear_proj.weight"], ws["linear_out.weight"])
        got = ff.forward(x.to(gpu), None).float().cpu()
        assert float((got - want).abs().max()) < (2e-5 if dtype == "float32" else 2e-2) * max(1.0, float(want.abs().max()))
    with pytest.raises(Exception, match="silu"):
        FEED_FORWARDS.build(PartSpec(kind="gated", hidden_size=8, intermediate_size=8, activation="gelu"), b)
    with pytest.raises(Exception, match="unknown norm kind"):
        NORMS.build(PartSpec(kind="layernorm", size=8), b)


# -- models from hand-written specs ---------------------------------------------------


def toy_spec(layers: dict, order: list, d=64, vocab=97, head_dim=16, rot=16, interleaved=False, max_pos=512,
             more_positions=None, ffs=None):
    norm = PartSpec(kind="rmsnorm", size=d, eps=1e-5)
    gated = PartSpec(kind="gated", hidden_size=d, intermediate_size=2 * d + 8, activation="silu")
    positions = {"rope": PartSpec(kind="rope", head_dim=head_dim, rotary_dim=rot, theta=10000.0,
                                  interleaved=interleaved, max_positions=max_pos)}
    positions.update(more_positions or {})
    return ModelSpec(
        architecture="toy", vocab_size=vocab, hidden_size=d, max_positions=max_pos,
        embedding=PartSpec(kind="embedding", vocab_size=vocab, size=d),
        positions=positions,
        layers={
            name: LayerSpec(mixer_norm=norm, mixer=mixer, ff_norm=norm, ff=(ffs or {}).get(name, gated))
            for name, mixer in layers.items()
        },
        order=order, final_norm=norm, head=PartSpec(kind="linear_head", vocab_size=vocab, size=d, tied=True),
    )


def attention_spec(d=64, heads=4, kv=2, head_dim=16, window=None, position="rope"):
    return PartSpec(kind="attention", hidden_size=d, n_heads=heads, n_kv_heads=kv, head_dim=head_dim,
                    scale=head_dim**-0.5, position=position, window=window)


def make_runner(gpu, spec, dtype, tokens=1024, page=16, **server):
    model = Decoder(spec, DT[dtype], gpu, tiled_weights=True)
    fill_random(model, seed=5, std=0.08)
    return ModelRunner(model, ServerConfig(kv_cache_num_tokens=tokens, page_size=page, max_seqs_per_forward=8, **server),
                       ModelConfig(dtype=dtype))


def plain_attention_layer(att, x, positions, rope_p, cached_kv=None):
    """One attention mixer from the plain functions; returns (output, (k, v))."""
    p = att.p
    w = att.w_qkv.float().cpu()
    nq, nk = p.n_heads * p.head_dim, p.n_kv_heads * p.head_dim
    n = x.shape[0]
    q = (x @ w[:nq].T).view(n, p.n_heads, p.head_dim)
    if p.position is not None:
        inv = P.inverse_frequencies(rope_p["rotary_dim"], rope_p["theta"])
        cos, sin = P.rotation_table(positions, inv)
        rotate = P.rotate_interleaved if rope_p["interleaved"] else P.rotate_half_split
        rot = rope_p["rotary_dim"]
        q = torch.cat((rotate(q[..., :rot], cos, sin), q[..., rot:]), -1)
    if cached_kv is None:
        k = (x @ w[nq : nq + nk].T).view(n, p.n_kv_heads, p.head_dim)
        v = (x @ w[nq + nk :].T).view(n, p.n_kv_heads, p.head_dim)
        if p.position is not None:
            k = torch.cat((rotate(k[..., :rot], cos, sin), k[..., rot:]), -1)
    else:
        k, v = cached_kv
    a = P.causal_attention(q, k, v, window=p.window)
    return a.reshape(n, nq) @ att.w_out.float().cpu().T, (k, v)


def plain_gated(ff, x):
    f = ff.p.intermediate_size
    wgu = ff.w_gate_up.float().cpu()
    return P.gated_feed_forward(x, wgu[:f], wgu[f:], ff.w_out.float().cpu())


def plain_model(model, ids, mixers: dict, ffs: dict | None = None):
    """The whole toy model from plain functions; ``mixers[layer name]`` is a function
    ``(mixer part, x, positions, run index, memo) -> delta``, ``ffs[layer name]`` a
    function ``(feed-forward part, x) -> delta`` (the gated one if none is given)."""
    spec = model.spec
    ids = torch.as_tensor(ids)
    positions = torch.arange(len(ids))
    h = P.embed(ids, model.embedding.weight.float().cpu())
    memo = {}
    for i, run in enumerate(spec.order):
        blk = model.layers[run.layer]
        parts = blk.parts()
        if isinstance(blk, SandwichBlock):
            h = plain_sandwich(parts, h, lambda x: mixers[run.layer](blk.mixer, x, positions, i, run, memo))
            continue
        x = P.rms_norm(h, parts["mixer_norm"].weight.float().cpu(), parts["mixer_norm"].p.eps)
        h = h + mixers[run.layer](blk.mixer, x, positions, i, run, memo)
        x = P.rms_norm(h, parts["ff_norm"].weight.float().cpu(), parts["ff_norm"].p.eps)
        h = h + (ffs or {}).get(run.layer, plain_gated)(parts["ff"], x)
    h = P.rms_norm(h, model.final_norm.weight.float().cpu(), model.final_norm.p.eps)
    return P.output_head(h, model.embedding.weight.float().cpu())


@register_arrangement("toy_sandwich")
class SandwichBlock(Arrangement):
    """Norms on both sides of the mixer, and a feed-forward that a layer may leave out:
    ``h += post_norm(mixer(pre_norm(h)))`` and then, if there is one, ``h += ff(ff_norm(h))``.
    Another set of parts than ``pre_norm`` has, under names of its own."""

    roles = {"pre_norm": NORMS, "mixer": MIXERS, "post_norm": NORMS, "ff_norm": NORMS, "ff": FEED_FORWARDS}
    optional = ("ff_norm", "ff")

    def forward(self, h, pending, ctx, run):
        p = self.parts()
        x = p["pre_norm"].forward(h, delta=pending)
        a = p["mixer"].forward(x, ctx, run)
        a = p["post_norm"].forward(a.float())  # a norm of the mixer's output, not of the stream
        if "ff" not in p:
            return a
        x = p["ff_norm"].forward(h, delta=a)
        return p["ff"].forward(x, ctx)


def plain_sandwich(parts, h, mixer):
    norm = lambda name, x: P.rms_norm(x, parts[name].weight.float().cpu(), parts[name].p.eps)  # noqa: E731
    h = h + norm("post_norm", mixer(norm("pre_norm", h)))
    if "ff" in parts:
        h = h + plain_gated(parts["ff"], norm("ff_norm", h))
    return h


def replay_all(runner, requests, ref, tol, vocab):
    for make in (replay.whole, replay.tail_one_by_one, replay.portions, replay.mixed):
        trace = make(requests)
        rows = replay.collect(trace, replay.run_trace(runner, trace), vocab)
        replay.compare(rows, ref, tol)
    assert runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_partial_rotation_and_a_layer_without_positions(gpu, dtype):
    """Three different mixers in one model: a window of 20 tokens with the adjacent
    pairing on half of the head, full attention, and attention without positions.
    The windowed layers have pages of their own, and give them back."""
    rope_p = dict(rotary_dim=8, theta=10000.0, interleaved=True)
    spec = toy_spec(
        {"win": attention_spec(window=20), "full": attention_spec(kv=4), "nopos": attention_spec(kv=1, position=None)},
        [LayerRun(layer="win"), LayerRun(layer="full"), LayerRun(layer="nopos"), LayerRun(layer="win")],
        rot=8, interleaved=True,
    )
    runner = make_runner(gpu, spec, dtype, tokens=640)
    assert len(runner.cache.groups) == 3 and runner.cache.groups[0].runs == [0, 3]

    def att(part, x, positions, i, run, memo):
        return plain_attention_layer(part, x, positions, rope_p)[0]

    requests = {f"r{i}": [int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 70 + i)] for i, n in enumerate([90, 33, 150, 7])}
    ref = {rid: plain_model(runner.model, toks, {"win": att, "full": att, "nopos": att}) for rid, toks in requests.items()}
    replay_all(runner, requests, ref, TOL[dtype], 97)
    # a long request holds only the window's pages in the windowed group
    s = runner.admit()
    runner.step([Segment(s, 0, requests["r2"], [])])
    win, full = runner.cache.groups[0], runner.cache.groups[1]
    assert sum(p >= 0 for p in win.tables[s]) <= 20 // 16 + 2 < sum(p >= 0 for p in full.tables[s]) == -(-150 // 16)
    runner.free(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_twice_and_a_borrowed_cache(gpu, dtype):
    """The run order names layer ``a`` twice (each run has a cache of its own) and
    lets the last run of ``b`` read the keys and values that run 1 wrote."""
    rope_p = dict(rotary_dim=16, theta=10000.0, interleaved=False)
    spec = toy_spec(
        {"a": attention_spec(), "b": attention_spec(heads=8, kv=2, head_dim=16)},
        [LayerRun(layer="a"), LayerRun(layer="b"), LayerRun(layer="a"), LayerRun(layer="b", cache_from=1)],
    )
    runner = make_runner(gpu, spec, dtype)
    assert sorted(runner.cache.group_of_run) == [0, 1, 2, 3]
    assert runner.model.runs[3].kv is runner.model.runs[1].kv and not runner.model.runs[3].appends
    assert runner.model.runs[2].kv is not runner.model.runs[0].kv

    def att(part, x, positions, i, run, memo):
        if run.cache_from is not None:
            return plain_attention_layer(part, x, positions, rope_p, cached_kv=memo[run.cache_from])[0]
        out, memo[i] = plain_attention_layer(part, x, positions, rope_p)
        return out

    requests = {f"r{i}": [int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 80 + i)] for i, n in enumerate([70, 5, 41])}
    ref = {rid: plain_model(runner.model, toks, {"a": att, "b": att}) for rid, toks in requests.items()}
    replay_all(runner, requests, ref, TOL[dtype], 97)


# -- a toy mixer with state of its own, defined and registered here ---------------------


class RunningMeanParams(BaseModel):
    hidden_size: int


@MIXERS.register("running_mean")
class RunningMean(Mixer):
    """``y_t = W * mean(x_0 .. x_t)``: no cache pages, but a per-request state (the sum
    so far and the count) that carries from one step to the next."""

    Params = RunningMeanParams

    def param_decls(self):
        return {"w.weight": ParamDecl((self.p.hidden_size, self.p.hidden_size))}

    def state_need(self):
        return {"sum": StateNeed((self.p.hidden_size,), torch.float32), "count": StateNeed((1,), torch.float32)}

    def forward(self, x, ctx, run):
        out = torch.empty_like(x, dtype=torch.float32)
        for seg, q0, n in zip(ctx.segments, ctx.seg_q_start_host, ctx.seg_q_len_host):
            xs = x[q0 : q0 + n].float()
            total = run.state["sum"][seg.slot] + torch.cumsum(xs, 0)
            count = run.state["count"][seg.slot] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)[:, None]
            out[q0 : q0 + n] = total / count
            run.state["sum"][seg.slot] = total[-1]
            run.state["count"][seg.slot] = count[-1]
        return (out @ self.w_weight.float().T).to(x.dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_mixer_with_state_is_registered_built_and_stepped(gpu, dtype):
    spec = toy_spec(
        {"mean": PartSpec(kind="running_mean", hidden_size=64), "att": attention_spec()},
        [LayerRun(layer="mean"), LayerRun(layer="att"), LayerRun(layer="mean")],
    )
    # the toy reads the step's slots on the host and does not say ``graph_safe``: asking for
    # graphs leaves this model on launches one by one
    runner = make_runner(gpu, spec, dtype, use_cudagraph=True)
    assert not runner.graphs_allowed
    assert len(runner.cache.groups) == 1 and runner.cache.groups[0].runs == [1]
    assert set(runner.cache.state.tensors) == {0, 2}  # each run of the layer has its own state rows
    rope_p = dict(rotary_dim=16, theta=10000.0, interleaved=False)

    def mean(part, x, positions, i, run, memo):
        m = torch.cumsum(x, 0) / torch.arange(1, x.shape[0] + 1)[:, None]
        return m @ part.w_weight.float().cpu().T

    def att(part, x, positions, i, run, memo):
        return plain_attention_layer(part, x, positions, rope_p)[0]

    requests = {f"r{i}": [int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 90 + i)] for i, n in enumerate([60, 3, 35, 18])}
    ref = {rid: plain_model(runner.model, toks, {"mean": mean, "att": att}) for rid, toks in requests.items()}
    replay_all(runner, requests, ref, TOL[dtype], 97)
    # a slot starts from zero again when the next request takes it
    s = runner.admit()
    assert float(runner.cache.state.tensors[0]["sum"][s].abs().sum()) == 0
    runner.free(s)


# -- a toy mixer whose pages hold one small vector a token, not keys and values -----------


@dataclass(frozen=True)
class LatentNeed(PagedNeed):
    width: int
    window: int | None = None

    def page_tensors(self, page_size):
        return {"latent": (page_size, self.width)}

    def bind(self, group_id, tensors, page_size, dtype):
        return LatentPages(group_id, tensors["latent"])


@dataclass
class LatentPages:
    group_id: int
    latent: torch.Tensor | None  # [pages, page_size, width]


class LookBackParams(BaseModel):
    hidden_size: int
    width: int
    window: int | None = None


@MIXERS.register("toy_look_back")
class ToyLookBack(Mixer):
    """``y_t = U * mean(D x_s for s in the last `window` tokens up to t)``: what it keeps of a
    token is ``D x_s``, ``width`` numbers, in pages of its own shape."""

    Params = LookBackParams

    def param_decls(self):
        p = self.p
        return {"down.weight": ParamDecl((p.width, p.hidden_size)), "up.weight": ParamDecl((p.hidden_size, p.width))}

    def cache_need(self):
        return LatentNeed(self.p.width, self.p.window)

    def forward(self, x, ctx, run):
        group = ctx.group(run.kv.group_id)
        pages, size = run.kv.latent, group.page_size
        latent = (x.float() @ self.down_weight.float().T).to(pages.dtype)
        out = torch.empty((x.shape[0], self.p.width), dtype=torch.float32, device=x.device)
        for i, (seg, q0, n) in enumerate(zip(ctx.segments, ctx.seg_q_start_host, ctx.seg_q_len_host)):
            table = group.block_table[i].long()
            now = torch.arange(seg.start, seg.start + n, device=x.device)
            pages[table[now // size], now % size] = latent[q0 : q0 + n]
            first = 0 if self.p.window is None else max(0, seg.start - self.p.window + 1)
            kept = torch.arange(first, seg.start + n, device=x.device)
            sums = torch.cumsum(pages[table[kept // size], kept % size].float(), 0)
            sums = torch.cat((torch.zeros_like(sums[:1]), sums))  # sums[j]: of the kept tokens before first + j
            lo = now - (self.p.window - 1) if self.p.window is not None else torch.zeros_like(now)
            lo = torch.clamp(lo, min=first)
            out[q0 : q0 + n] = (sums[now + 1 - first] - sums[lo - first]) / (now + 1 - lo)[:, None]
        return (out @ self.up_weight.float().T).to(x.dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_mixer_with_pages_of_another_shape(gpu, dtype):
    spec = toy_spec(
        {"far": PartSpec(kind="toy_look_back", hidden_size=64, width=24), "att": attention_spec(),
         "near": PartSpec(kind="toy_look_back", hidden_size=64, width=24, window=20)},
        [LayerRun(layer="far"), LayerRun(layer="att"), LayerRun(layer="near"), LayerRun(layer="far")],
    )
    runner = make_runner(gpu, spec, dtype, tokens=192)
    cache = runner.cache
    assert [g.runs for g in cache.groups] == [[0, 3], [1], [2]]
    pages = cache.num_pages
    assert cache.groups[0].storage.shape == (2, pages * 16 * 24) and cache.groups[2].storage.shape == (1, pages * 16 * 24)
    assert cache.groups[1].storage.shape == (1, pages * 2 * 2 * 16 * 16)
    needs = {i: runner.model.mixer_of_run(i).cache_need() for i in range(4)}
    assert cache.bytes_per_page(needs, 16, DT[dtype]) == (3 * 16 * 24 + 2 * 2 * 16 * 16) * DT[dtype].itemsize
    assert runner.model.runs[0].kv.latent.data_ptr() != runner.model.runs[3].kv.latent.data_ptr()
    for g in cache.groups:  # a page that was never written, or is read after its time, shows
        g.storage.fill_(float("nan"))
    rope_p = dict(rotary_dim=16, theta=10000.0, interleaved=False)
    round_to = (lambda t: t.to(torch.bfloat16).float()) if dtype == "bfloat16" else (lambda t: t)

    def look_back(part, x, positions, i, run, memo):
        latent = round_to(x @ part.down_weight.float().cpu().T)
        w = part.p.window or x.shape[0]
        mean = torch.stack([latent[max(0, t - w + 1) : t + 1].mean(0) for t in range(x.shape[0])])
        return mean @ part.up_weight.float().cpu().T

    def att(part, x, positions, i, run, memo):
        return plain_attention_layer(part, x, positions, rope_p)[0]

    requests = {f"r{i}": [int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 70 + i)] for i, n in enumerate([60, 3, 35, 18])}
    ref = {rid: plain_model(runner.model, toks, {"far": look_back, "near": look_back, "att": att}) for rid, toks in requests.items()}
    replay_all(runner, requests, ref, TOL[dtype], 97)
    # the windowed group gives pages back while a request runs, the other keeps them
    slot = runner.admit()
    runner.step([Segment(slot, 0, requests["r0"][:50], want=[])])
    held = [sum(p >= 0 for p in g.tables[slot]) for g in cache.groups]
    assert held == [4, 4, 3], held  # the next query looks back to token 31, on the second page
    runner.free(slot)
    assert cache.idle()


# -- a toy feed-forward that routes, and another position encoding ------------------------


class RoutedParams(BaseModel):
    hidden_size: int
    n_experts: int
    expert_size: int


@FEED_FORWARDS.register("toy_routed")
class ToyRouted(FeedForward):
    """Each token goes to the expert with the largest router logit (float32 logits and
    softmax); the expert is ``W2 silu(W1 x)`` and its output is weighted with the
    router's probability."""

    Params = RoutedParams

    def param_decls(self):
        p = self.p
        return {
            "router.weight": ParamDecl((p.n_experts, p.hidden_size)),
            "w1.weight": ParamDecl((p.n_experts, p.expert_size, p.hidden_size)),
            "w2.weight": ParamDecl((p.n_experts, p.hidden_size, p.expert_size)),
        }

    def forward(self, x, ctx):
        probs = torch.softmax(x.float() @ self.router_weight.float().T, dim=-1)
        weight, expert = probs.max(dim=-1)
        out = torch.zeros_like(x, dtype=torch.float32)
        for e in range(self.p.n_experts):
            rows = torch.nonzero(expert == e)[:, 0]
            if rows.numel():
                hid = torch.nn.functional.silu(x[rows].float() @ self.w1_weight[e].float().T)
                out[rows] = (hid @ self.w2_weight[e].float().T) * weight[rows, None]
        return out.to(x.dtype)


def plain_routed(ff, x):
    router, w1, w2 = (t.float().cpu() for t in (ff.router_weight, ff.w1_weight, ff.w2_weight))
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        probs = torch.softmax(x[t] @ router.T, dim=-1)
        e = int(probs.argmax())
        out[t] = probs[e] * (w2[e] @ torch.nn.functional.silu(w1[e] @ x[t]))
    return out


class SinusoidParams(BaseModel):
    size: int
    base: float


@POSITIONS.register("toy_sinusoid")
class ToySinusoid(PositionEncoding):
    """Absolute positions as a vector of sines and cosines that a mixer adds to its input."""

    Params = SinusoidParams

    def encode(self, positions):
        half = self.p.size // 2
        freq = self.p.base ** (-torch.arange(half, device=positions.device, dtype=torch.float32) / half)
        ang = positions.float()[:, None] * freq[None, :]
        return torch.cat((torch.sin(ang), torch.cos(ang)), dim=-1)


class AddPositionParams(BaseModel):
    hidden_size: int
    position: str


@MIXERS.register("toy_add_position")
class ToyAddPosition(Mixer):
    """``y = W (x + encode(position))`` with the position encoding that the model's
    specification names: no cache and no state, only the step's positions."""

    Params = AddPositionParams

    def __init__(self, params, build):
        super().__init__(params, build)
        self.position = build.positions[params.position]

    def param_decls(self):
        return {"w.weight": ParamDecl((self.p.hidden_size, self.p.hidden_size))}

    def forward(self, x, ctx, run):
        y = x.float() + self.position.encode(ctx.positions)
        return (y @ self.w_weight.float().T).to(x.dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routing_and_other_position_encodings(gpu, dtype):
    """One model with: attention under a second rotary encoding (other base, adjacent
    pairs, part of the head), a mixer that uses a position encoding defined here, a
    feed-forward with routing in one layer and the gated one in the others."""
    rope_a = dict(rotary_dim=16, theta=10000.0, interleaved=False)
    rope_b = dict(rotary_dim=8, theta=300.0, interleaved=True)
    spec = toy_spec(
        {"a": attention_spec(), "b": attention_spec(kv=1, position="rope_b"),
         "pos": PartSpec(kind="toy_add_position", hidden_size=64, position="sin")},
        [LayerRun(layer="a"), LayerRun(layer="pos"), LayerRun(layer="b")],
        more_positions={
            "rope_b": PartSpec(kind="rope", head_dim=16, rotary_dim=8, theta=300.0, interleaved=True, max_positions=512),
            "sin": PartSpec(kind="toy_sinusoid", size=64, base=50.0),
        },
        ffs={"b": PartSpec(kind="toy_routed", hidden_size=64, n_experts=3, expert_size=40)},
    )
    runner = make_runner(gpu, spec, dtype)
    assert isinstance(runner.model.layers["b"].parts()["ff"], ToyRouted)
    assert not isinstance(runner.model.layers["a"].parts()["ff"], ToyRouted)

    def att_with(rope_p):
        return lambda part, x, positions, i, run, memo: plain_attention_layer(part, x, positions, rope_p)[0]

    def add_position(part, x, positions, i, run, memo):
        half = 32
        ang = positions.float()[:, None] * (50.0 ** (-torch.arange(half, dtype=torch.float32) / half))[None, :]
        return (x + torch.cat((torch.sin(ang), torch.cos(ang)), -1)) @ part.w_weight.float().cpu().T

    requests = {f"r{i}": [int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 120 + i)] for i, n in enumerate([50, 4, 37])}
    mixers = {"a": att_with(rope_a), "b": att_with(rope_b), "pos": add_position}
    ref = {rid: plain_model(runner.model, toks, mixers, {"b": plain_routed}) for rid, toks in requests.items()}
    replay_all(runner, requests, ref, TOL[dtype], 97)


# -- an arrangement that knows nothing of the norms folded into products ----------------



@register_arrangement("pre_norm_plain_test")
class PlainPreNorm(Arrangement):
    """The same arithmetic as ``pre_norm`` through the plain interface: four parts, tensors
    in, a tensor out, no word about the block before or after."""

    roles = {"mixer_norm": NORMS, "mixer": MIXERS, "ff_norm": NORMS, "ff": FEED_FORWARDS}

    def forward(self, h, pending, ctx, run):
        p = self.parts()
        x = p["mixer_norm"].forward(h, delta=pending)
        assert isinstance(x, torch.Tensor) and (pending is None or isinstance(pending, torch.Tensor))
        a = p["mixer"].forward(x, ctx, run)
        x = p["ff_norm"].forward(h, delta=a)
        assert isinstance(a, torch.Tensor) and isinstance(x, torch.Tensor)
        return p["ff"].forward(x, ctx)


def test_a_plain_arrangement_between_blocks_that_fold_their_norms(gpu):
    """``pre_norm`` blocks fold their norms into the products around them where both sides can;
    a block with the plain interface in between is handed tensors only, and the model gives
    what the plain implementation gives."""
    rope_p = dict(rotary_dim=16, theta=10000.0, interleaved=False)
    spec = toy_spec({"a": attention_spec(), "b": attention_spec(heads=2, kv=1), "c": attention_spec(kv=4)},
                    [LayerRun(layer="a"), LayerRun(layer="b"), LayerRun(layer="c"), LayerRun(layer="a")])
    spec.layers["b"].arrangement = "pre_norm_plain_test"
    runner = make_runner(gpu, spec, "bfloat16")

    def att(part, x, positions, i, run, memo):
        return plain_attention_layer(part, x, positions, rope_p)[0]

    requests = {f"r{i}": [int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 60 + i)] for i, n in enumerate([50, 3, 35])}
    ref = {rid: plain_model(runner.model, toks, {"a": att, "b": att, "c": att}) for rid, toks in requests.items()}
    replay_all(runner, requests, ref, TOL["bfloat16"], 97)


# -- another set of parts in a block ----------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_arrangement_with_other_parts_is_registered_from_here(gpu, dtype):
    """A block with norms before and after its mixer, once with and once without a
    feed-forward, between two ``pre_norm`` blocks: described as data, built and stepped
    with no change to the framework."""
    rope_p = dict(rotary_dim=16, theta=10000.0, interleaved=False)
    spec = toy_spec({"a": attention_spec(), "s": attention_spec(heads=2, kv=1), "t": attention_spec(kv=4)},
                    [LayerRun(layer="a"), LayerRun(layer="s"), LayerRun(layer="t"), LayerRun(layer="a")])
    norm = spec.final_norm
    spec.layers["s"] = LayerSpec(arrangement="toy_sandwich", parts=dict(
        pre_norm=norm, mixer=spec.layers["s"].parts["mixer"], post_norm=norm, ff_norm=norm, ff=spec.layers["s"].parts["ff"]))
    spec.layers["t"] = LayerSpec(arrangement="toy_sandwich", parts=dict(
        pre_norm=norm, mixer=spec.layers["t"].parts["mixer"], post_norm=norm))
    spec = ModelSpec(**spec.model_dump())  # the description is data
    runner = make_runner(gpu, spec, dtype)
    assert sorted(runner.model.layers["t"].parts()) == ["mixer", "post_norm", "pre_norm"]
    names = {s.path for s in runner.model.param_slots()}
    assert "layers.s.post_norm.weight" in names and "layers.t.ff.linear_out.weight" not in names

    def att(part, x, positions, i, run, memo):
        return plain_attention_layer(part, x, positions, rope_p)[0]

    requests = {f"r{i}": [int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 70 + i)] for i, n in enumerate([50, 3, 35])}
    ref = {rid: plain_model(runner.model, toks, {"a": att, "s": att, "t": att}) for rid, toks in requests.items()}
    replay_all(runner, requests, ref, TOL[dtype], 97)
    with pytest.raises(Exception, match=r"leaves out \['post_norm'\]"):
        bad = spec.model_copy(deep=True)
        del bad.layers["t"].parts["post_norm"]
        Decoder(bad, DT[dtype], gpu)


# -- toy models under the scheduler ------------------------------------------------------------


def greedy_with_plain_model(model, mixers, prompt, n_new):
    ids, out = list(prompt), []
    for _ in range(n_new):
        t = int(torch.argmax(plain_model(model, ids, mixers)[-1]))
        out.append(t)
        ids.append(t)
    return out


@pytest.mark.parametrize("ahead", [0, 1])
def test_the_scheduler_serves_a_model_without_paged_layers(gpu, ahead):
    """Every layer keeps state of fixed size and none keeps keys: no group of pages exists,
    slots are the only limit, prompts are cut into portions and requests wait for a slot."""
    from halite_amd.engine import InferenceEngine

    spec = toy_spec({"m": PartSpec(kind="running_mean", hidden_size=64), "n": PartSpec(kind="running_mean", hidden_size=64)},
                    [LayerRun(layer="m"), LayerRun(layer="n"), LayerRun(layer="m")])
    model = Decoder(spec, torch.float32, gpu)
    fill_random(model, seed=5, std=0.08)
    runner = ModelRunner(model, ServerConfig(page_size=16, max_seqs_per_forward=2, max_tokens_per_forward=16,
                                             chunked_prefill_size=7, scheduling_steps_ahead=ahead), ModelConfig(dtype="float32"))
    assert runner.cache.groups == []
    engine = InferenceEngine(runner)

    def mean(part, x, positions, i, run, memo):
        return (torch.cumsum(x, 0) / torch.arange(1, x.shape[0] + 1)[:, None]) @ part.w_weight.float().cpu().T

    prompts = [[int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 30 + n)] for n in (23, 2, 9, 40)]
    results = engine.infer_batch([(i, p, {"max_new_tokens": 6, "temperature": 0.0}) for i, p in enumerate(prompts)])
    for r, p in zip(results, prompts):
        assert r.output_ids[0] == greedy_with_plain_model(model, {"m": mean, "n": mean}, p, 6)
    st = engine.stats
    assert st.max_running == 2 and st.retractions == 0 and max(st.tokens_per_step) <= 16
    assert runner.cache.idle()


@pytest.mark.parametrize("ahead", [0, 1])
def test_the_scheduler_serves_two_groups_of_pages_and_retracts(gpu, ahead):
    """Layers with a window beside layers with all keys, each kind with pages of its own, and
    so few pages that requests are retracted: the tokens are those of the plain model, and
    the retractions come in bursts with headroom, not one per step."""
    from halite_amd.engine import InferenceEngine

    rope_p = dict(rotary_dim=16, theta=10000.0, interleaved=False)
    spec = toy_spec({"w": attention_spec(window=12), "f": attention_spec(kv=1)},
                    [LayerRun(layer="w"), LayerRun(layer="f"), LayerRun(layer="w")])
    model = Decoder(spec, torch.float32, gpu)
    fill_random(model, seed=6, std=0.08)
    runner = ModelRunner(model, ServerConfig(kv_cache_num_tokens=152, page_size=8, max_seqs_per_forward=8,
                                             max_tokens_per_forward=24, chunked_prefill_size=10,
                                             default_init_new_token_ratio=0.05, retract_decode_steps=6,
                                             scheduling_steps_ahead=ahead), ModelConfig(dtype="float32"))
    assert len(runner.cache.groups) == 2
    engine = InferenceEngine(runner)

    def att(part, x, positions, i, run, memo):
        return plain_attention_layer(part, x, positions, rope_p)[0]

    prompts = [[int(t) % 97 for t in tiny.random_tokens(tiny.TINY_A, n, 50 + n)] for n in (21, 5, 13, 30)]
    results = engine.infer_batch([(i, p, {"max_new_tokens": 24, "temperature": 0.0}) for i, p in enumerate(prompts)])
    for r, p in zip(results, prompts):
        assert r.output_ids[0] == greedy_with_plain_model(model, {"w": att, "f": att}, p, 24)
    st = engine.stats
    assert 0 < st.retractions <= 6, st.retractions
    assert runner.cache.idle()
    runner.cache.check()


# -- a whole toy architecture, from config.json keys of its own to generated tokens --------


class ToyMixConfig(BaseModel):
    """The keys of the toy's config.json; nothing of it is known to the framework."""

    architectures: list[str]
    width: int
    vocab: int
    kinds: list[str]  # per layer: "mean" (the running mean above) or "attention"
    heads: int
    kv_heads: int
    head_size: int
    inner: int
    eps: float
    theta: float
    context: int
    window: int | None = None  # of the attention layers after the first
    torch_dtype: str | None = None


def toy_mix_spec(cfg: ToyMixConfig) -> ModelSpec:
    norm = PartSpec(kind="rmsnorm", size=cfg.width, eps=cfg.eps)
    ff = PartSpec(kind="gated", hidden_size=cfg.width, intermediate_size=cfg.inner, activation="silu")
    layers, seen_attention = {}, False
    for i, kind in enumerate(cfg.kinds):
        if kind == "mean":
            mixer = PartSpec(kind="running_mean", hidden_size=cfg.width)
        else:
            mixer = PartSpec(kind="attention", hidden_size=cfg.width, n_heads=cfg.heads, n_kv_heads=cfg.kv_heads,
                             head_dim=cfg.head_size, scale=cfg.head_size**-0.5, position="rope",
                             window=cfg.window if seen_attention else None)
            seen_attention = True
        layers[f"L{i}"] = LayerSpec(arrangement="pre_norm", parts=dict(mixer_norm=norm, mixer=mixer, ff_norm=norm, ff=ff))
    return ModelSpec(
        architecture="ToyMixForCausalLM", vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.context,
        embedding=PartSpec(kind="embedding", vocab_size=cfg.vocab, size=cfg.width),
        positions={"rope": PartSpec(kind="rope", head_dim=cfg.head_size, rotary_dim=cfg.head_size, theta=cfg.theta,
                                    interleaved=False, max_positions=cfg.context)},
        layers=layers, order=[LayerRun(layer=name) for name in layers], final_norm=norm,
        head=PartSpec(kind="linear_head", vocab_size=cfg.vocab, size=cfg.width, tied=True),
    )


def toy_mix_weight_map(cfg: ToyMixConfig) -> dict:
    # one table for both kinds of layer: a layer takes the names of the parameters it has
    return {
        "toy.table": "embedding.weight",
        "toy.#.before_mixer": "layers.#.mixer_norm.weight",
        "toy.#.mean": "layers.#.mixer.w.weight",
        "toy.#.q": "layers.#.mixer.q.weight",
        "toy.#.k": "layers.#.mixer.k.weight",
        "toy.#.v": "layers.#.mixer.v.weight",
        "toy.#.o": "layers.#.mixer.out.weight",
        "toy.#.before_ff": "layers.#.ff_norm.weight",
        "toy.#.gate": "layers.#.ff.linear_gate.weight",
        "toy.#.up": "layers.#.ff.linear_proj.weight",
        "toy.#.down": "layers.#.ff.linear_out.weight",
        "toy.last_norm": "final_norm.weight",
    }


TOY_MIX = dict(architectures=["ToyMixForCausalLM"], width=64, vocab=211, kinds=["mean", "attention", "attention", "mean"],
               heads=4, kv_heads=2, head_size=16, inner=88, eps=1e-5, theta=10000.0, context=256, window=24)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_architecture_from_its_config_file_to_generated_tokens(gpu, dtype, tmp_path, capsys):
    """An architecture of its own (config keys, layer kinds that differ from layer to layer,
    tensor names) is registered here; the framework's folder writer, loader, engine,
    scheduler and sampler then serve it as they serve the built-in one."""
    import json

    from halite_amd.config.registry import Architecture, register_architecture
    from halite_amd.engine.engine import InferenceEngine
    from halite_amd.weights import WeightError
    from halite_amd.weights.random_init import write_random_model

    arch = register_architecture(Architecture("ToyMixForCausalLM", ToyMixConfig, toy_mix_spec, toy_mix_weight_map))
    try:
        found, cfg = parse_config(dict(TOY_MIX))
        assert found is arch and cfg.kinds == TOY_MIX["kinds"]
        folder = write_random_model(str(tmp_path / "toy"), cfg, seed=3, dtype=dtype, std=0.08)
        with open(f"{folder}/config.json") as f:
            assert json.load(f)["kinds"] == TOY_MIX["kinds"]
        server = ServerConfig(kv_cache_num_tokens=512, page_size=16, max_seqs_per_forward=4, chunked_prefill_size=16,
                              max_tokens_per_forward=32, max_prefill_tokens=32)
        engine = InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype=dtype))
        model = engine.model_runner.model
        assert [type(model.layers[n].mixer).__name__ for n in model.spec.layers] == ["RunningMean", "Attention", "Attention", "RunningMean"]
        assert len(engine.model_runner.cache.groups) == 2  # all keys; a window of them
        rope_p = dict(rotary_dim=16, theta=10000.0, interleaved=False)

        def mean(part, x, positions, i, run, memo):
            return (torch.cumsum(x, 0) / torch.arange(1, x.shape[0] + 1)[:, None]) @ part.w_weight.float().cpu().T

        def att(part, x, positions, i, run, memo):
            return plain_attention_layer(part, x, positions, rope_p)[0]

        mixers = {"L0": mean, "L1": att, "L2": att, "L3": mean}
        prompts = [[int(t) % 211 for t in tiny.random_tokens(tiny.TINY_A, n, 60 + n)] for n in (41, 3, 70)]
        results = engine.infer_batch([(p, {"max_new_tokens": 12, "temperature": 0.0}) for p in prompts])
        margin = 1e-4 if dtype == "float32" else 0.06
        for p, r in zip(prompts, results):
            out = r.output_ids[0]
            assert len(out) == 12
            logits = plain_model(model, p + out, mixers)
            for j, tok in enumerate(out):  # the chosen token is the plain model's best, or within rounding of it
                row = logits[len(p) - 1 + j]
                assert float(row.max() - row[tok]) <= margin * max(1.0, float(row.abs().max())), (len(p), j)
        assert engine.stats.prefill_tokens >= sum(len(p) for p in prompts) and engine.model_runner.cache.idle()
        # the command line draws random prompts from the toy's vocabulary, which its
        # configuration calls by a name of its own
        from halite_amd.cli import generate as command_line

        capsys.readouterr()
        status = command_line.main(["--model", folder, "--prompt-lens", "9,4", "--prompt-seed", "2", "sampling.temperature=0",
                                    "sampling.max_new_tokens=3", f"model.dtype={dtype}", "server.kv_cache_num_tokens=256",
                                    "server.max_seqs_per_forward=4"])
        lines = [json.loads(line) for line in capsys.readouterr().out.strip().split("\n")]
        assert status == 0 and [len(r["input_ids"]) for r in lines] == [9, 4]
        assert all(0 <= t < 211 for r in lines for t in r["input_ids"] + r["output_ids"][0])
        # the loader's one error speaks the toy's tensor names
        from safetensors import safe_open
        from safetensors.torch import save_file

        with safe_open(f"{folder}/model.safetensors", "pt") as f:
            tensors = {k: f.get_tensor(k) for k in f.keys()}
        tensors.pop("toy.L0.mean")
        tensors["toy.L3.q"] = torch.zeros(2, 2)
        save_file(tensors, f"{folder}/model.safetensors")
        with pytest.raises(WeightError) as e:
            InferenceEngine.from_pretrained(folder, server, ModelConfig(dtype=dtype))
        assert "toy.L0.mean" in str(e.value) and "toy.L3.q" in str(e.value)
    finally:
        from halite_amd.config.registry import ARCHITECTURES

        ARCHITECTURES.pop("ToyMixForCausalLM", None)
