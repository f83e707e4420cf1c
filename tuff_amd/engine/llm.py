"""The Python entry point: from prompts (token ids) to generated token ids.

    llm = LLM("model_dir", dtype="bfloat16")
    outs = llm.generate([[1, 36309]], SamplingParams(max_new_tokens=16))

`generate` is the reference's run loop (prefill in portions, then one token a step until -n
tokens, src/main.c:1743-1858) for many requests at once: scheduler -> step -> sampler.
"""
from __future__ import annotations

import dataclasses
import itertools
from typing import Optional, Sequence

import torch

from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .engine import Engine, StepFailed
from .scheduler import PLACEHOLDER, Request, Scheduler


@dataclasses.dataclass
class Generation:
    request_id: object
    prompt: list
    token_ids: list
    finish_reason: str
    preemptions: int = 0


class LLM:
    def __init__(self, model=None, *, engine: Optional[Engine] = None, dtype="bfloat16", device="cuda:0",
                 max_num_seqs: int = 8, max_batched_tokens: int = 2048, ctx_size: Optional[int] = None,
                 page_size: int = 16, num_pages: Optional[int] = None, ignore_eos: bool = False,
                 run_ahead: bool = True):
        """model: a folder with config.json and model.safetensors.  ctx_size (-c): the longest
        prompt + generation of one request.  num_pages: size of the page pool; default: room for
        max_num_seqs requests of ctx_size."""
        if engine is None:
            if model is None:
                raise ValueError("give a model folder or an engine")
            from ..models.registry import load_config
            cfg = load_config(model)
            limit = getattr(cfg, "max_position_embeddings", None)
            ctx = min(ctx_size or 4096, limit or (ctx_size or 4096))
            pages = num_pages if num_pages is not None else max_num_seqs * -(-ctx // page_size)
            engine = Engine.from_folder(model, dtype=dtype, device=device, page_size=page_size,
                                        num_pages=pages, max_requests=max_num_seqs)
            ctx_size = ctx
        self.engine = engine
        model_limit = engine.model.max_positions
        self.ctx_size = min(c for c in (ctx_size, model_limit) if c is not None) if (ctx_size or model_limit) else None
        self.max_num_seqs = min(max_num_seqs, engine.manager.num_slots)
        self.max_batched_tokens = max_batched_tokens
        self.ignore_eos = ignore_eos
        self.run_ahead = run_ahead
        self.sampler = Sampler(engine.device)
        self._ids = itertools.count()
        self.last_stats: dict = {}

    def new_scheduler(self) -> Scheduler:
        eos = None if self.ignore_eos else self.engine.model.eos_token_id
        return Scheduler(self.engine.manager, begin=self.engine.begin, end=self.engine.end,
                         max_num_seqs=self.max_num_seqs, max_batched_tokens=self.max_batched_tokens,
                         max_model_len=self.ctx_size, eos_token_id=eos)

    def run(self, sched: Scheduler, on_step=None) -> None:
        """Steps until every request of the scheduler has finished."""
        loop = Loop(self, sched)
        while True:
            done = loop.step()
            if done is None:
                break
            if on_step is not None:
                on_step(*done)
        self.last_stats = loop.stats()

    def generate(self, prompts: Sequence[Sequence[int]], params=None, inputs=None) -> list[Generation]:
        """prompts: token id lists.  params: one SamplingParams for all, or one per prompt.  inputs: for a
        model whose parts read more of a token than its id and position, one function a prompt (or None),
        inputs[i](start, n) -> {name: integers [n] or [n, cols]} for the tokens at places start .. start + n - 1
        of prompt i and what is generated after it (scheduler.Request.inputs)."""
        if params is None:
            params = SamplingParams()
        plist = [params] * len(prompts) if isinstance(params, SamplingParams) else list(params)
        if len(plist) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        ilist = [None] * len(prompts) if inputs is None else list(inputs)
        if len(ilist) != len(prompts):
            raise ValueError("one inputs function per prompt (or None)")
        sched = self.new_scheduler()
        reqs = []
        for prompt, p, more in zip(prompts, plist, ilist):
            r = Request(next(self._ids), [int(t) for t in prompt], dataclasses.replace(p), inputs=more)
            reqs.append(r)
            sched.add(r)
        self.run(sched)
        return [Generation(r.id, r.prompt, list(r.output), r.finish_reason or "", r.preemptions) for r in reqs]


class Loop:
    """The run loop, one step a call: scheduler -> step -> sampler -> scheduler.

    The next step is decided and started before the tokens of the current one have reached the
    host (`run_ahead`): a request that decodes takes its token from the sampler's output on the
    device.  The host then decides, packs and accounts while the GPU runs.  Not where the next
    step would have to preempt somebody, and not while a sampler needs the tokens on the host
    (a penalty over the request's history).
    Requests may be added to the scheduler between calls."""

    def __init__(self, llm: "LLM", sched: Scheduler):
        self.llm, self.sched = llm, sched
        self.under_way = None                             # a step started ahead: (batch, sampling, pending)
        self.steps = self.tokens = self.ahead_steps = 0

    def _start(self, batch, before=None):
        """before: (requests that draw a token in the step before, its sampler launch)."""
        entries, places, sources, at = [], [], [], 0
        row = {id(r): i for i, r in enumerate(before[0])} if before is not None else {}
        for s in batch:
            toks = s.tokens
            if PLACEHOLDER in toks:
                if len(toks) != 1 or before is None:
                    raise RuntimeError("a token that is not known yet can only be fed alone, and from the step before")
                places.append(at)
                sources.append(row[id(s.request)])
                toks = [0]
            more = s.request.inputs(s.start, len(toks)) if s.request.inputs is not None else None
            entries.append(StepEntry(s.request.id, toks, [len(toks) - 1] if s.samples else [], more))
            at += len(toks)
        device_tokens = None
        if places:
            out = before[1].out
            whole = len(places) == at == out.shape[0] and sources == places
            device_tokens = out if whole else (out, places, sources)
        logits = self.llm.engine.step(entries, device_tokens)
        sampling = [s.request for s in batch if s.samples]
        pending = self.llm.sampler.launch(logits, [r.sampler for r in sampling]) if sampling else None
        return sampling, pending

    def _end_requests_of(self, failed: StepFailed) -> None:
        """What the requests of a step that failed midway hold is gone: they end here, with the reason, and give
        back their pages and slots.  The scheduler's other requests go on if the caller calls again."""
        for rid in failed.requests:
            self.sched.abort(rid, reason=f"error: {failed.__cause__}")

    def step(self):
        """Runs one step and accounts for it.  Returns (the Scheduled entries whose requests were
        still live, {request id: token drawn}), or None when nothing is left to do."""
        sched, sampler = self.sched, self.llm.sampler
        if self.under_way is None:
            if not sched.has_unfinished():
                return None
            batch = sched.schedule()
            if not batch:
                if sched.has_unfinished():
                    raise RuntimeError("the scheduler made no progress: no request fits the cache")
                return None
            try:
                sampling, pending = self._start(batch)
            except StepFailed as e:
                self._end_requests_of(e)
                raise
        else:
            batch, sampling, pending = self.under_way
            self.under_way = None
        live = sched.advance(batch)
        failed = None
        if self.llm.run_ahead and not any(sampler.needs_history(r.sampler) for r in sampling):
            nxt = sched.schedule(ahead=True)
            if nxt:
                try:
                    self.under_way = (nxt,) + self._start(nxt, (sampling, pending))
                    self.ahead_steps += 1
                except StepFailed as e:
                    failed = e                             # this step's own tokens are still accounted for below
        sampled = {}
        if pending is not None:
            sampled = {r.id: t for r, t in zip(sampling, pending.tokens())}
        sched.commit(batch, sampled)
        if failed is not None:
            self._end_requests_of(failed)                  # after commit(): their last tokens are in place
            raise failed
        self.steps += 1
        self.tokens += sum(len(s.tokens) for s in live)
        return live, {s.request.id: sampled[s.request.id] for s in live if s.samples}

    def stats(self) -> dict:
        return {"steps": self.steps, "tokens_run": self.tokens, "preemptions": self.sched.num_preemptions,
                "steps_started_ahead": self.ahead_steps}
