"""The step function and what it owns: the model, the cache manager, the staging.

``ModelRunner.step`` takes a batch of (request slot, its next tokens, the places whose
logits are wanted), portions of prompts beside single decoded tokens, cut anywhere; it
runs exactly those tokens as one batch from the cache that earlier steps left, and
returns float32 logits at the wanted places.  The reference has one runner per engine
(src/halite/transformers/infer/engine/model_runner.py:14-252) with separate extend and
decode passes; the mixed flat batch is the ``tokainfer`` engine's
(src/halite/transformers/tokainfer/basic_worker.py:56-174).
"""

from __future__ import annotations

import gc

import numpy as np
import torch

from ..cache import CacheManager, NoSpace
from ..config.engine import ModelConfig, ServerConfig, check_stated_sizes
from ..config.registry import read_config
from ..parts.decoder import Decoder
from ..weights import fill_random, load_weights
from ..kernels import attention as attention_kernels
from ..kernels import ops
from .batch import Segment, StaticLayout, StepContext, _Staging

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class StepError(ValueError):
    pass


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError(
            "halite_amd runs on an AMD GPU through its HIP kernels only; no GPU is visible "
            f"(device {device}) and there is no CPU path"
        )
    return device


class ModelRunner:
    def __init__(
        self,
        model: Decoder,
        server_config: ServerConfig | None = None,
        model_config: ModelConfig | None = None,
    ):
        self.model = model
        self.server_config = server_config or ServerConfig()
        self.model_config = model_config or ModelConfig(
            dtype="float32" if model.dtype == torch.float32 else "bfloat16"
        )
        self.device = model.device
        spec = model.spec
        self.context_len = min(self.model_config.context_len or spec.max_positions, spec.max_positions)
        self.vocab_size = spec.vocab_size

        needs, borrowed, state_needs = {}, {}, {}
        for i, run in enumerate(spec.order):
            mixer = model.mixer_of_run(i)
            need = mixer.cache_need()
            if need is not None:
                if run.cache_from is None:
                    needs[i] = need
                else:
                    borrowed[i] = run.cache_from
            st = mixer.state_need()
            if st:
                state_needs[i] = st
        sizes = [model.mixer_of_run(i).attention_sizes() for i in range(len(spec.order))]
        check_stated_sizes(self.model_config, len(spec.order), [s for s in sizes if s is not None])
        page_size = self.server_config.page_size
        n_slots = self.server_config.max_seqs_per_forward
        num_pages = self._size_pool(needs, page_size, model.dtype)
        self.cache = CacheManager(
            needs, borrowed, state_needs, page_size=page_size, num_pages=num_pages,
            n_slots=n_slots, dtype=model.dtype, device=self.device,
        )
        for run in model.runs:
            run.kv = self.cache.layer_pages(run.index)
            run.state = self.cache.state_of_run(run.index)
        self._staging = _Staging(self.device) if self.device.type == "cuda" else None
        self.max_total_tokens = self.cache.token_capacity
        # position tables for the whole context, so that their addresses never change
        for pos in model.positions.values():
            if hasattr(pos, "tables"):
                pos.tables(self.context_len)
        self._graphs: dict[int, dict] = {}  # batch size -> layout and recorded decode step
        self._ahead = None  # (requests and positions, cache version, context) of a step put together ahead
        self._pages_taken_ahead: set[int] = set()  # slots for which such steps reserved and may not have come
        self.steps_taken_ahead = 0
        self._token_feed = None
        # graphs replay a model only if every part of it reads what varies on the device
        self.graphs_allowed = (
            self.server_config.use_cudagraph and self.device.type == "cuda"
            and all(p.graph_safe for p in self.model.named_parts().values())
            and all(b.graph_safe for b in self.model.layers.values())
        )
        self.graph_replays = 0
        self.released = False
        self.has_weights = True  # the model comes filled; restore() gives one that is not

    def _size_pool(self, needs, page_size, dtype) -> int:
        tokens = self.server_config.kv_cache_num_tokens
        if tokens is not None:
            return -(-tokens // page_size) + 1
        if not needs:
            return 2
        # src/halite/transformers/infer/engine/model_runner.py:117-131
        free, total = torch.cuda.mem_get_info(self.device)
        usable = free - total * (1 - self.model_config.memory_fraction_static)
        per_page = CacheManager.bytes_per_page(needs, page_size, dtype)
        pages = int(usable // per_page)
        if pages < 2:
            raise RuntimeError("no device memory is left for the cache pool")
        # a request never holds more than context_len tokens; cap the pool at what
        # max_seqs_per_forward requests of that length could use
        cap = self.server_config.max_seqs_per_forward * (-(-self.context_len // page_size)) + 1
        return min(pages, cap)

    # -- construction -------------------------------------------------------------
    @staticmethod
    def _want_tiled(spec, dtype, device, server_config) -> bool:
        mode = (server_config or ServerConfig()).decode_weight_copy
        if dtype != torch.bfloat16 or mode == "off":
            return False
        if mode == "on":
            return True
        probe = Decoder(spec, dtype, "cpu")
        _, total = torch.cuda.mem_get_info(device)
        return 2 * probe.param_bytes() < total / 3

    @classmethod
    def from_pretrained(cls, folder: str, server_config=None, model_config=None) -> "ModelRunner":
        model_config = model_config or ModelConfig()
        device = require_gpu(f"{model_config.device}:{model_config.gpu_id}" if model_config.device == "cuda" else model_config.device)
        arch, cfg = read_config(folder)
        spec, dtype = arch.to_spec(cfg), _TORCH_DTYPE[model_config.dtype]
        model = Decoder(spec, dtype, device, cls._want_tiled(spec, dtype, device, server_config))
        load_weights(model, arch.weight_map(cfg), folder)
        runner = cls(model, server_config, model_config)
        runner.arch, runner.config = arch, cfg
        return runner

    @classmethod
    def from_random(cls, cfg, seed: int, server_config=None, model_config=None, arch=None) -> "ModelRunner":
        from ..config.registry import get_architecture

        model_config = model_config or ModelConfig()
        device = require_gpu(f"{model_config.device}:{model_config.gpu_id}" if model_config.device == "cuda" else model_config.device)
        arch = arch or get_architecture(cfg.architectures[0])
        spec, dtype = arch.to_spec(cfg), _TORCH_DTYPE[model_config.dtype]
        model = Decoder(spec, dtype, device, cls._want_tiled(spec, dtype, device, server_config))
        fill_random(model, seed)
        runner = cls(model, server_config, model_config)
        runner.arch, runner.config = arch, cfg
        return runner

    def load_state_dict(self, tensors: dict) -> None:
        """New weights from tensors in memory, named as in a model folder.  The requests
        that are live keep their cache; captured graphs hold the old tensors and are
        dropped."""
        from ..weights import load_state_dict

        if self.released:
            raise RuntimeError("the runner was released; restore() it before weights are loaded")
        load_state_dict(self.model, self.arch.weight_map(self.config), tensors)
        self._graphs.clear()
        self._ahead = None
        self.has_weights = True

    def release(self) -> None:
        """Gives the device memory back: captured graphs, the cache pool and the state
        rows, the weights and their tiled copies, the position tables (the reference's
        engine frees its pools and moves the model to the meta device so that a trainer
        can have the GPU, src/halite/transformers/infer/engine/engine.py:43-46;
        model_runner.py:241-252).  ``restore`` makes the runner usable again."""
        if self.released:
            return
        if not self.cache.idle():
            raise RuntimeError("requests are still live; free them before the runner is released")
        self._graphs.clear()
        self._ahead = self._token_feed = self._staging = None
        for run in self.model.runs:
            run.kv, run.state = None, {}
        self.cache.release_storage()
        holders = list(self.model.named_parts().values()) + list(self.model.positions.values())
        for part in holders:
            for name, value in list(vars(part).items()):
                if isinstance(value, torch.Tensor):
                    setattr(part, name, None)
        self.released, self.has_weights = True, False
        gc.collect()
        if self.device.type == "cuda":
            torch.cuda.empty_cache()

    def restore(self) -> None:
        """After ``release``: a cache pool of the configured size again, and the model's
        tensors allocated but not filled; ``load_state_dict`` brings the weights."""
        if not self.released:
            return
        spec, dtype, tiled = self.model.spec, self.model.dtype, self.model.build.tiled_weights
        arch, config = getattr(self, "arch", None), getattr(self, "config", None)
        self.__init__(Decoder(spec, dtype, self.device, tiled), self.server_config, self.model_config)
        self.has_weights = False
        if arch is not None:
            self.arch, self.config = arch, config

    # -- requests -------------------------------------------------------------------
    def admit(self) -> int:
        return self.cache.admit()

    def free(self, slot: int) -> None:
        self.cache.free(slot)

    def capture_graphs(self, batch_sizes=None) -> list[int]:
        """Records the decode graphs of the given batch sizes now instead of at their
        first use (the reference records its graphs when the engine is set up,
        src/halite/transformers/infer/engine/model_runner.py:159-239); without sizes,
        those that the server configuration lists (``cudagraph_additonal_batch_size`` and
        the multiples of ``cudagraph_step``).  Needs an idle cache: every size is run
        once with one-token requests that are freed again.  Returns the sizes that have
        a graph afterwards."""
        if not self.graphs_allowed:
            return []
        if not self.cache.idle():
            raise RuntimeError("graphs are recorded ahead of time only while no request is live")
        most = min(self.server_config.cudagraph_max_batch_size, self.server_config.max_seqs_per_forward)
        if batch_sizes is None:
            cfg = self.server_config
            batch_sizes = set(cfg.cudagraph_additonal_batch_size) | set(range(cfg.cudagraph_step, most + 1, cfg.cudagraph_step))
        for b in sorted(set(batch_sizes)):
            entry = self._graphs.get(b)
            if b < 1 or b > most or (entry is not None and entry["graph"] is not None):
                continue
            slots = [self.admit() for _ in range(b)]
            try:
                self.step([Segment(slot, 0, [0], [0]) for slot in slots])
            except NoSpace:
                break  # the pool is smaller than this many pages: larger sizes cannot occur
            finally:
                for slot in slots:
                    self.free(slot)
        self._ahead = None
        return sorted(b for b, e in self._graphs.items() if e["graph"] is not None)

    # -- the step ---------------------------------------------------------------------
    def check_segments(self, segments: list[Segment], n_ids: int | None = None) -> None:
        n_ids = self.vocab_size if n_ids is None else n_ids
        seen = set()
        for s in segments:
            if s.slot in seen:
                raise StepError(f"slot {s.slot} appears twice in one step")
            seen.add(s.slot)
            n = s.tokens.size
            if n == 0:
                raise StepError(f"slot {s.slot}: an entry without tokens")
            have = self.cache.length(s.slot)
            if s.start != have:
                raise StepError(f"slot {s.slot}: tokens start at {s.start} but {have} are cached")
            if s.start + n > self.context_len:
                raise StepError(f"slot {s.slot}: {s.start + n} tokens exceed the context length {self.context_len}")
        every = np.concatenate([s.tokens for s in segments]) if len(segments) > 1 else segments[0].tokens
        if int(every.min()) < 0 or int(every.max()) >= n_ids:
            for s in segments:
                lo, hi = int(s.tokens.min()), int(s.tokens.max())
                if lo < 0 or hi >= n_ids:
                    raise StepError(f"slot {s.slot}: token id {lo if lo < 0 else hi} outside the vocabulary of {n_ids}")

    @torch.no_grad()
    def step(self, segments: list[Segment], token_feed=None) -> torch.Tensor:
        """Runs the tokens of ``segments`` and returns float32 logits
        ``[wanted rows, vocab]`` in the order of the segments and of their ``want``.
        Raises ``NoSpace`` (and changes nothing) if the pages do not suffice.

        ``token_feed``: int32 token ids on the device (what an earlier step sampled and
        the host has not read yet).  Every segment then has one token, and
        ``segments[i].tokens[0]`` is not a token id but the row of ``token_feed`` that
        holds it."""
        if self.released or not self.has_weights:
            raise RuntimeError("the runner has no weights on the device (released, or restored and not loaded)")
        if not segments:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        if token_feed is not None and any(s.tokens.size != 1 for s in segments):
            raise StepError("tokens can be fed on the device only to segments of one token")
        self._token_feed = token_feed
        self.check_segments(segments, self.vocab_size if token_feed is None else token_feed.numel())
        spans = [(s.slot, s.start + s.tokens.size) for s in segments]
        graph_step = (
            self.graphs_allowed
            and len(segments) <= self.server_config.cudagraph_max_batch_size
            and all(s.tokens.size == 1 and s.want == [0] for s in segments)
        )
        ahead = self._take_step_ahead(segments) if graph_step else None
        if ahead is None:  # a step that was put together ahead has its pages already
            try:
                self.cache.reserve(spans)
            except NoSpace:
                # pages may be held for a step that was prepared ahead and is not the one that came
                if not self._release_pages_taken_ahead():
                    raise
                self.cache.reserve(spans)
        else:
            self._pages_taken_ahead.difference_update(s.slot for s in segments)
        logits = None
        try:
            if graph_step:
                logits = self._step_graph(segments, ahead)
            if logits is None:
                ctx = StepContext(segments, self.cache, self.device, self._staging)
                for run in self.model.runs:
                    self.model.mixer_of_run(run.index).prepare(ctx, run)
                self._feed_tokens(ctx)
                logits = self.model.forward(ctx)
        except BaseException:
            # a step that stops half-way may leave pieces counted that nobody merged
            attention_kernels.reset_counters(self.device)
            raise
        for slot, new_len in spans:
            self.cache.advance(slot, new_len)
        if graph_step:
            self._put_step_ahead(segments)
        return logits

    def _feed_tokens(self, ctx) -> None:
        """Token ids that are still on the device go straight into the step's array, whose
        entries name their rows until then."""
        feed, self._token_feed = self._token_feed, None
        if feed is not None:
            ops.take_tokens(feed, ctx.tokens)

    # While the GPU works on a decode step, the host puts the next one together as far as
    # it can without the tokens: the same requests, one position on.  If that is what
    # the next call brings (and nothing else touched the cache meanwhile), only the token
    # ids are filled in.
    def _put_step_ahead(self, segments: list[Segment]) -> None:
        self._ahead = None
        entry = self._graphs.get(len(segments))
        if entry is None or entry["graph"] is None:
            return
        nxt = [Segment(s.slot, s.start + 1, [0], [0]) for s in segments]
        if any(s.start + 1 > self.context_len for s in nxt):
            return
        try:
            self.cache.reserve([(s.slot, s.start + 1) for s in nxt])
        except NoSpace:
            return
        self._pages_taken_ahead.update(s.slot for s in nxt)
        ctx = StepContext(nxt, self.cache, self.device, self._staging, static=entry["layout"])
        for run in self.model.runs:
            self.model.mixer_of_run(run.index).prepare(ctx, run)
        self._ahead = (tuple((s.slot, s.start) for s in nxt), self.cache.version, ctx)

    def _release_pages_taken_ahead(self) -> bool:
        """Gives back the pages of the step that was prepared ahead; whether any came back."""
        slots, self._pages_taken_ahead = self._pages_taken_ahead, set()
        live = self.cache.slots.live()
        return sum(self.cache.release_unused(s) for s in slots if s in live) > 0

    def _take_step_ahead(self, segments: list[Segment]):
        ahead, self._ahead = self._ahead, None
        if ahead is None:
            return None
        key, version, ctx = ahead
        if version != self.cache.version or key != tuple((s.slot, s.start) for s in segments):
            return None
        ctx.replace_tokens(np.concatenate([s.tokens for s in segments]))
        self.steps_taken_ahead += 1
        return ctx

    def _step_graph(self, segments: list[Segment], ahead=None):
        """A decode-only step through a captured HIP graph, one graph per batch size
        (the reference captures its decode pass per padded batch size,
        src/halite/transformers/infer/engine/model_runner.py:159-239).  The step's
        arrays live in one persistent buffer that is refilled before every replay;
        the kernels' grids are sized for the layout's capacities and read the live
        counts from that buffer.  The first step of a batch size runs eagerly and
        records the graph; the returned logits are overwritten by the next replay."""
        B = len(segments)
        entry = self._graphs.get(B)
        if entry is None:
            width = {g.group_id: -(-self.context_len // g.page_size) for g in self.cache.groups}
            entry = self._graphs[B] = {"layout": StaticLayout(B, width, self.device), "graph": None}
        ctx = ahead
        if ctx is None:
            ctx = StepContext(segments, self.cache, self.device, self._staging, static=entry["layout"])
            for run in self.model.runs:
                self.model.mixer_of_run(run.index).prepare(ctx, run)
        if not ctx.fits_static():
            return None
        ctx.upload()
        self._feed_tokens(ctx)
        if entry["graph"] is None:
            logits = self.model.forward(ctx)  # this step, for real
            graph = torch.cuda.CUDAGraph()
            # No garbage collection while the stream records: a graph of an engine that
            # is no longer used would be destroyed in the middle of it, which HIP refuses.
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph):
                    entry["logits"] = self.model.forward(ctx)  # recorded, not run
            finally:
                if collecting:
                    gc.enable()
            entry["graph"], entry["ctx"] = graph, ctx
            return logits
        entry["graph"].replay()
        self.graph_replays += 1
        return entry["logits"]
