"""The engine: a bound model, its cache, and the one step function.

`step(entries)` takes, for each request in the step, its next tokens (a portion of a prompt of
any length, or one decoded token) and the places whose logits are wanted.  It runs exactly
those tokens as one batch against the cache that earlier steps left and returns the float32
logits of the wanted places.  The reference's counterparts take one token or up to eight
consecutive tokens of its single request (src/lfm25_engine.c:434-475, :496-599).
"""
from __future__ import annotations

import math
from typing import Hashable, Optional, Sequence

import torch

from ..cache.manager import CacheLayout, CacheManager, OutOfPages
from ..cache.storage import CacheStorage
from ..config.base import ModelConfig
from ..csrc import ops
from ..models.registry import build_model, load_config
from ..parts.base import Runtime
from ..weights.loader import load_weights
from ..weights.random_init import random_weights
from .batch import StepContext, StepEntry, build_context, check_token_inputs, context_on, pack_step

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
           "fp32": torch.float32, "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine computes in bfloat16 or float32, not {name}")
        return name
    if name not in _DTYPES:
        raise ValueError(f"unknown dtype '{name}'; choose bfloat16 or float32")
    return _DTYPES[name]


def require_gpu(device="cuda:0") -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: this engine runs its model on a gfx950 GPU through its "
                           "own HIP kernels and has no CPU path")
    return torch.device(device)


class StepFailed(RuntimeError):
    """A step failed after its kernels had begun to run (a launch that was refused, an error in a part).
    `.requests`: the ids of the step's requests; what they hold is no longer consistent (a fixed-size state has
    moved on for some layers, pages that a window had passed are gone) and the engine refuses further steps of
    them: end() them.  Requests that were not in the step are untouched."""

    def __init__(self, requests, cause):
        self.requests = list(requests)
        super().__init__(f"the step failed midway ({type(cause).__name__}: {cause}); its requests "
                         f"{self.requests} must be ended")


class Engine:
    def __init__(self, model, weights: dict, *, dtype, device="cuda:0", page_size: int = 16,
                 max_tokens: int = 8192, max_requests: int = 8, num_pages=None, poison_cache: bool = False,
                 use_graphs: bool = True):
        """max_tokens: tokens the page pool of each cache group holds (rounded up to whole
        pages).  max_requests: state slots, i.e. requests that can be live at a time."""
        self.device = require_gpu(device)
        self.dtype = parse_dtype(dtype)
        self.model = model
        self.rt = Runtime(self.device, self.dtype)
        for m in model.kernel_modules() + (["gemm_f32"] if self.dtype == torch.float32 else ["gemm_bf16"]):
            ops.load(m)                      # compile or load now, not in the middle of a step
        model.bind(weights, self.rt)
        # what the parts read of a step's tokens beside ids and positions (StepEntry.inputs brings it)
        self.token_inputs = tuple(model.token_inputs()) if hasattr(model, "token_inputs") else ()
        self.layout = CacheLayout.from_specs(model.cache_specs)
        self.page_size = int(page_size)
        if num_pages is None:
            num_pages = -(-int(max_tokens) // self.page_size)
        self.manager = CacheManager(self.layout, self.page_size, num_pages, int(max_requests))
        self.storage = CacheStorage(self.manager, self.dtype, self.device, poison=poison_cache)
        self.steps = 0
        self._broken: set = set()            # requests of a step that failed midway: no further steps, only end()
        # steps of single decoded tokens are recorded into graphs, one per (batch size, table width)
        # (nothing is recorded while the kernel classes are being timed: events cannot go into a graph)
        self.use_graphs = bool(use_graphs) and model.graph_safe() and not ops.TRACE
        self._graphs: dict = {}
        self.graph_replays = 0
        self.record_portions = self.use_graphs and model.records_portions()
        self._sectioned: dict = {}
        self._sectioned_seen: dict = {}
        self._record_at = self.SECTIONS_RECORD_AT
        self._calm_replays = 0
        self.section_replays = 0
        self.section_recordings = 0

    # ---------------------------------------------------------------- construction
    @classmethod
    def from_folder(cls, model_dir: str, *, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        dev = require_gpu(device)
        cfg = load_config(model_dir)
        model = build_model(cfg)
        weights = load_weights(model_dir, model.weight_decls(), parse_dtype(dtype), dev)
        eng = cls(model, weights, dtype=dtype, device=device, **kw)
        eng.config = cfg
        return eng

    @classmethod
    def from_config(cls, cfg: ModelConfig, seed: int, *, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        """Random weights made on the device (no folder is written)."""
        dev = require_gpu(device)
        model = build_model(cfg)
        weights = random_weights(model.weight_decls(), seed, parse_dtype(dtype), dev)
        eng = cls(model, weights, dtype=dtype, device=device, **kw)
        eng.config = cfg
        return eng

    # -------------------------------------------------------------------- requests
    def begin(self, req_id: Hashable) -> None:
        slot = self.manager.admit(req_id)
        self.storage.zero_slot(slot)

    def end(self, req_id: Hashable) -> None:
        self.manager.release(req_id)
        self._broken.discard(req_id)

    def is_live(self, req_id) -> bool:
        return req_id in self.manager

    def length(self, req_id) -> int:
        return self.manager.length(req_id)

    # ------------------------------------------------------------------------ step
    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Runs one batch.  Returns float32 logits [wanted, vocab] on the device, in the order
        of the entries and of their `want` lists, or None if nothing is wanted.  The tensor may be the
        step function's own buffer (a recorded step writes its logits to the same place at every replay):
        it holds this step's logits until the next step; a caller that keeps them copies them.
        Raises OutOfPages (and leaves every request as it was) if the pool is too small.
        device_tokens: for a caller that starts a step before it has seen the last one's tokens.
        Either an int32 tensor on the device with one id per token of the step, or a triple
        (tensor, places, sources): token `places[i]` of the step is `tensor[sources[i]]`.  The ids
        are put in place by a kernel on the stream; the entries' ids at those places only stand in."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        entries = [e for e in entries if len(e.tokens) > 0]
        if not entries:
            return None
        ids = [e.req_id for e in entries]
        if len(set(ids)) != len(ids):
            raise ValueError("a request appears twice in one step")
        limit = self.model.max_positions
        V = self.model.vocab_size
        for e in entries:                     # refuse bad input before anything is changed
            if e.req_id not in self.manager:
                raise ValueError(f"request {e.req_id!r} is not live: call begin() first")
            if e.req_id in self._broken:
                raise ValueError(f"request {e.req_id!r} was in a step that failed midway: what it holds is not "
                                 f"consistent any more, end() it")
            if min(e.tokens) < 0 or max(e.tokens) >= V:
                raise ValueError(f"request {e.req_id!r}: token id outside [0, {V})")
            if any((not 0 <= w < len(e.tokens)) for w in e.want):
                raise ValueError(f"request {e.req_id!r}: a wanted place is outside its {len(e.tokens)} tokens")
        check_token_inputs(entries, self.token_inputs)
        done = []
        try:
            for e in entries:
                if limit is not None and self.manager.length(e.req_id) + len(e.tokens) > limit:
                    raise ValueError(f"request {e.req_id!r} would pass the model's {limit} positions")
                self.manager.extend(e.req_id, len(e.tokens))
                done.append(e)
        except Exception:
            for e in done:
                self.manager.truncate(e.req_id, self.manager.length(e.req_id) - len(e.tokens))
            raise
        if device_tokens is not None:
            n = sum(len(e.tokens) for e in entries)
            try:
                device_tokens = self._check_device_tokens(device_tokens, n)
            except ValueError:
                for e in done:
                    self.manager.truncate(e.req_id, self.manager.length(e.req_id) - len(e.tokens))
                raise
        try:
            out = self._run(entries, device_tokens)
        except Exception as exc:
            # A launch that was refused, or an error in a part, after some kernels ran.  The book-keeping goes back
            # to before the step so that pages and lengths stay sound, but the requests' contents do not: a
            # fixed-size state of a layer that did run has moved on, and pages that fell out of a window when the
            # step was accounted are gone (freed, and filled with NaN under poison_cache).  So the step's requests
            # are refused from now on; all the caller can do with them is end().
            for e in done:
                self.manager.truncate(e.req_id, self.manager.length(e.req_id) - len(e.tokens))
                self._broken.add(e.req_id)
            raise StepFailed([e.req_id for e in done], exc) from exc
        self.steps += 1
        return out

    def _run(self, entries, device_tokens):
        if self.use_graphs and all(len(e.tokens) == 1 for e in entries):
            return self._decode_step(entries, device_tokens)
        ctx = build_context(entries, self.manager, self.device, self.model.vocab_size, self.token_inputs)
        # Recorded in sections: steps with portions (a step of single tokens takes other kernels), keyed by
        # everything their launches depend on outside of the sections that run eagerly.
        if (self.record_portions and ctx.T >= self.SECTIONS_MIN_TOKENS and ctx.max_q_len > 1
                and ctx.R <= self.manager.num_slots):
            return self._portion_step(ctx, device_tokens)
        self._place_device_tokens(ctx.tokens, device_tokens)
        return self.model.forward(ctx, self.storage.views)

    def _check_device_tokens(self, device_tokens, n: int):
        """A tensor of all n ids stays; a triple becomes (tensor, index tensor [places | sources])."""
        if isinstance(device_tokens, torch.Tensor):
            if device_tokens.dtype != torch.int32 or device_tokens.shape != (n,) or device_tokens.device != self.device:
                raise ValueError(f"device_tokens must be int32 [{n}] on {self.device}")
            return device_tokens
        src, places, sources = device_tokens
        if src.dtype != torch.int32 or src.dim() != 1 or src.device != self.device or len(places) != len(sources):
            raise ValueError(f"device_tokens: an int32 vector on {self.device} and as many places as sources are needed")
        if any(not 0 <= p < n for p in places) or any(not 0 <= q < src.shape[0] for q in sources):
            raise ValueError("device_tokens: a place or a source is out of range")
        if not places:
            return None
        idx = torch.tensor(list(places) + list(sources), dtype=torch.int32).pin_memory().to(self.device, non_blocking=True)
        return src, idx

    @staticmethod
    def _place_device_tokens(tokens: torch.Tensor, device_tokens) -> None:
        if device_tokens is None:
            return
        if isinstance(device_tokens, torch.Tensor):
            tokens.copy_(device_tokens)
        else:
            ops.scatter_i32(tokens, device_tokens[0], device_tokens[1])

    # ------------------------------------------------------- steps recorded in sections
    SECTIONS_MIN_TOKENS = 2          # every step with a portion may be recorded (a step of 64 tokens: 1.57 ms of launches, 1.22 ms replayed)
    SECTIONS_RECORD_AT = 3           # a number of tokens is recorded when it comes for this time (more, once sizes push each other out)
    MAX_SECTIONED = 4
    SECTIONS_CALM_REPLAYS = 64       # so many replays without a recording pushed out unused: the threshold halves again
    SECTIONS_SEEN_KEPT = 256         # sizes whose counts are kept (the least recently seen go first)

    def _portion_step(self, ctx, device_tokens=None) -> Optional[torch.Tensor]:
        """A step with prompt portions.  What its kernels' launches depend on outside of the
        sections that parts run eagerly (ctx.run_eagerly) is what the model's recording_key() names (the
        number of tokens, and whether the last block prepares the head's norm), so a step shape that
        keeps coming (a scheduler fills its budget) is recorded once: graphs
        of the stretches between those sections, replayed with the sections run in between."""
        key = self.model.recording_key(ctx)
        rec = self._sectioned.get(key)
        if rec is None:
            seen = self._sectioned_seen.pop(key, 0) + 1    # (taken out and put back: the most recently seen is last)
            self._sectioned_seen[key] = seen
            while len(self._sectioned_seen) > self.SECTIONS_SEEN_KEPT:
                self._sectioned_seen.pop(next(iter(self._sectioned_seen)))      # came once or twice, long ago
            if seen < self._record_at:
                self._place_device_tokens(ctx.tokens, device_tokens)
                return self.model.forward(ctx, self.storage.views)
            if len(self._sectioned) >= self.MAX_SECTIONED:
                torch.cuda.synchronize()                    # its last replay may still be under way
                old_key = next(iter(self._sectioned))
                if self._sectioned.pop(old_key).replays <= 1:
                    # More sizes take turns than recordings are kept: this one was pushed out before it was
                    # used again.  Recording costs about two eager steps, so sizes now have to come more often.
                    self._record_at = min(2 * self._record_at, 1 << 16)
                    self._sectioned_seen[old_key] = 0
                    self._calm_replays = 0
            self.section_recordings += 1
            rec = _SectionedStep(ctx.T, self.manager.num_slots, self.device)
            try:
                rec.record(ctx, lambda c: self.model.forward(c, self.storage.views))
            except Exception as e:                         # noqa: BLE001 - recording is an optimisation
                import sys
                print(f"[tuff_amd] recording a step of {ctx.T} tokens in sections failed "
                      f"({type(e).__name__}: {e}); continuing without", file=sys.stderr)
                self.record_portions = False
                self._sectioned.clear()
                self._place_device_tokens(ctx.tokens, device_tokens)
                return self.model.forward(ctx, self.storage.views)
            self._sectioned[key] = rec
        else:
            self._sectioned[key] = self._sectioned.pop(key)           # most recently used last
        merged = rec.refresh(ctx)
        self._place_device_tokens(merged.tokens, device_tokens)
        self.section_replays += 1
        # A phase of many sizes (ragged tails of prompts) raises the threshold; once the sizes that come are replayed
        # again and again without one being pushed out unused, it comes down, or a later steady stream of another
        # size would never be recorded.
        self._calm_replays += 1
        if self._calm_replays >= self.SECTIONS_CALM_REPLAYS and self._record_at > self.SECTIONS_RECORD_AT:
            self._record_at = max(self.SECTIONS_RECORD_AT, self._record_at // 2)
            self._calm_replays = 0
        return rec.replay(merged)

    # --------------------------------------------------------------- recorded decode
    GRAPH_TABLE_BUCKET = 64          # block tables of recorded steps are padded to multiples of this
    MAX_GRAPHS = 12

    def _decode_step(self, entries, device_tokens=None) -> Optional[torch.Tensor]:
        """A step of single tokens.  The first step of a shape runs eagerly on persistent
        buffers and is then recorded; later steps of that shape refresh the buffer and replay.
        Everything a kernel's launch depends on (batch size, table width, number of key
        partitions) is part of the shape; positions, tokens, tables and slots are data."""
        longest = max([len(self.manager.block_table(e.req_id, g)) for e in entries
                       for g in range(len(self.manager.groups))] + [1])
        width = -(-longest // self.GRAPH_TABLE_BUCKET) * self.GRAPH_TABLE_BUCKET
        p = pack_step(entries, self.manager, self.model.vocab_size, max_blocks=width, token_inputs=self.token_inputs)
        key = p.shape_key()
        g = self._graphs.get(key)
        if g is None:
            if len(self._graphs) >= self.MAX_GRAPHS:
                torch.cuda.synchronize()                    # its last replay may still be under way
                self._graphs.pop(next(iter(self._graphs)))
            g = _RecordedStep(p, self.device, width * self.page_size)
            g.refresh(p, device_tokens)
            logits = self.model.forward(g.ctx, self.storage.views)
            self._graphs[key] = g                           # only a shape whose eager step went through
            try:
                g.record(lambda: self.model.forward(g.ctx, self.storage.views))
            except Exception as e:                         # noqa: BLE001 - recording is an optimisation
                import sys
                print(f"[tuff_amd] recording the decode step failed ({type(e).__name__}: {e}); "
                      f"continuing without graphs", file=sys.stderr)
                self.use_graphs = False
                self._graphs.clear()
            return logits
        self._graphs[key] = self._graphs.pop(key)           # most recently used last
        g.refresh(p, device_tokens)
        g.graph.replay()
        self.graph_replays += 1
        return g.logits


class _SectionedStep:
    """A step of T tokens recorded as graphs with eager sections between them.

    What the graphs read of the step lies in one persistent buffer, [tokens T | req_of_token T |
    q_start | q_len | state_slot], the three per-request arrays padded to the most requests a step
    can hold (q_len 0 beyond the step's own); every other field of a step's context is the step's own.
    """

    def __init__(self, T: int, max_requests: int, device):
        self.T, self.R = T, max_requests
        n = 2 * T + 3 * max_requests
        self.pinned = torch.empty(n, dtype=torch.int32, pin_memory=True)
        self.dev = torch.empty(n, dtype=torch.int32, device=device)
        self.copied = torch.cuda.Event()
        self.pool = torch.cuda.graph_pool_handle()
        self.program: list = []                # graphs and functions of a context, in order
        self.replays = 0
        self._graph = None
        self._capture = None

    def _views(self):
        T, R, d = self.T, self.R, self.dev
        return dict(tokens=d[:T], req_of_token=d[T:2 * T], q_start=d[2 * T:2 * T + R],
                    q_len=d[2 * T + R:2 * T + 2 * R], state_slot=d[2 * T + 2 * R:2 * T + 3 * R])

    def refresh(self, ctx):
        """Brings the persistent buffer up to this step (one copy on the stream, out of what the
        step's own context was packed from) and returns the step's context over it."""
        import dataclasses
        T, R, r = self.T, self.R, ctx.R
        packed = ctx.host["packed"]
        self.copied.synchronize()                           # the last copy out of `pinned` is done
        buf = self.pinned.numpy()
        buf[:T] = packed["tokens"]
        buf[T:2 * T] = packed["req_of_token"]
        buf[2 * T:] = 0
        buf[2 * T:2 * T + r] = packed["q_start"]
        buf[2 * T + R:2 * T + R + r] = packed["q_len"]
        buf[2 * T + 2 * R:2 * T + 2 * R + r] = packed["state_slot"]
        self.dev.copy_(self.pinned, non_blocking=True)
        self.copied.record()
        return dataclasses.replace(ctx, **self._views())

    # -- recording: nothing runs; the eager sections are only noted
    def _begin(self) -> None:
        self._graph = torch.cuda.CUDAGraph()
        self._capture = torch.cuda.graph(self._graph, pool=self.pool)
        self._capture.__enter__()

    def _end(self) -> None:
        import warnings
        with warnings.catch_warnings(record=True) as caught:
            warnings.simplefilter("always")
            self._capture.__exit__(None, None, None)
        if not any("Graph is empty" in str(w.message) for w in caught):    # e.g. nothing after the last section
            self.program.append(self._graph)
        self._graph = self._capture = None

    def eager(self, fn) -> None:
        self._end()
        self.program.append(fn)
        self._begin()

    def record(self, ctx, forward) -> None:
        import dataclasses
        merged = dataclasses.replace(ctx, recorder=self, host=dict(ctx.host), **self._views())
        torch.cuda.synchronize()
        self._begin()
        try:
            forward(merged)
        except BaseException:
            self._capture.__exit__(None, None, None)
            self._graph = self._capture = None
            raise
        self._end()

    def replay(self, ctx):
        out = None
        self.replays += 1
        for piece in self.program:
            if isinstance(piece, torch.cuda.CUDAGraph):
                piece.replay()
            else:
                out = piece(ctx)
        return out


class _RecordedStep:
    """Persistent buffers of one step shape and the graph recorded over them."""

    def __init__(self, p, device, max_ctx_len: int):
        self.pinned = torch.empty(p.buf.size, dtype=torch.int32, pin_memory=True)
        self.dev = torch.empty(p.buf.size, dtype=torch.int32, device=device)
        self.ctx = context_on(self.dev, p, max_ctx_len=max_ctx_len)
        self.copied = torch.cuda.Event()
        self.graph = None
        self.logits = None

    def refresh(self, p, device_tokens=None) -> None:
        self.copied.synchronize()                           # the last copy out of `pinned` is done
        self.pinned.numpy()[:] = p.buf
        self.dev.copy_(self.pinned, non_blocking=True)
        self.copied.record()
        Engine._place_device_tokens(self.ctx.tokens, device_tokens)

    def record(self, forward) -> None:
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.logits = forward()
        self.graph = graph
