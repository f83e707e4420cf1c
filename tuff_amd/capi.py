"""The Python half of the plain C interface (include/tuff_amd.h).

The C library calls these functions with integers: handles of sessions kept here, and the
addresses of the caller's arrays, which are read and written in place through ctypes.  The
structures below mirror the header field by field.  Everything else is the engine's ordinary
Python entry point: Engine.step for tuff_engine_step, Scheduler and Loop for the tuff_sched
calls, LLM.generate for tuff_generate.
"""
from __future__ import annotations

import ctypes as C
import itertools
import json

FINISH_CODES = {"stop": 1, "length": 2, "context": 3, "capacity": 4, "aborted": 5}
FINISH_REJECTED = 6


class CSampling(C.Structure):
    _fields_ = [("temp", C.c_float), ("top_p", C.c_float), ("top_k", C.c_int32), ("min_p", C.c_float),
                ("repeat_penalty", C.c_float), ("repeat_last_n", C.c_int32), ("seed", C.c_uint64),
                ("max_new_tokens", C.c_int32), ("ignore_eos", C.c_int32)]


class CStepEntry(C.Structure):
    _fields_ = [("request", C.c_int64), ("tokens", C.POINTER(C.c_int32)), ("n_tokens", C.c_int32),
                ("want", C.POINTER(C.c_int32)), ("n_want", C.c_int32)]


class CEvent(C.Structure):
    _fields_ = [("request", C.c_int64), ("token", C.c_int32), ("finished", C.c_int32)]


def struct_sizes() -> tuple:
    """(sizeof tuff_sampling, tuff_step_entry, tuff_event) as this module lays them out; the C
    library compares them with its own at start."""
    return C.sizeof(CSampling), C.sizeof(CStepEntry), C.sizeof(CEvent)


def _params(addr: int):
    from .sampling.params import SamplingParams
    if not addr:
        return SamplingParams()
    s = CSampling.from_address(addr)
    return SamplingParams(temp=s.temp, top_p=s.top_p, top_k=s.top_k, min_p=s.min_p,
                          repeat_penalty=s.repeat_penalty, repeat_last_n=s.repeat_last_n, seed=s.seed,
                          max_new_tokens=s.max_new_tokens, ignore_eos=bool(s.ignore_eos))


def _ints(addr, n: int) -> list:
    if n < 0:
        raise ValueError("a negative count")
    if n == 0:
        return []
    if not addr:
        raise ValueError("a null array with a positive count")
    return list((C.c_int32 * n).from_address(addr if isinstance(addr, int) else C.addressof(addr.contents)))


class Session:
    """One loaded engine with its scheduler for the tuff_sched calls.  The caller's request
    numbers are kept apart from each other and from LLM.generate's own: ("step", n) for requests
    of tuff_request_begin, ("sched", n) for those of tuff_request_add."""

    def __init__(self, model_dir: str, dtype: str, max_requests: int, ctx_size: int):
        from .engine.llm import LLM, Loop
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype '{dtype}': bfloat16 or float32")
        if max_requests < 1:
            raise ValueError("max_requests must be positive")
        self.llm = LLM(model_dir, dtype=dtype, max_num_seqs=max_requests, ctx_size=ctx_size or None)
        self.engine = self.llm.engine
        self.sched = self.llm.new_scheduler()
        self.loop = Loop(self.llm, self.sched)
        self.requests: dict = {}
        self.reported = 0                 # requests of sched.finished already reported

    # -- step function
    def step(self, entries_addr: int, n: int, logits_addr: int, capacity: int) -> int:
        from .engine.batch import StepEntry
        if n < 1 or not entries_addr:
            raise ValueError("a step needs at least one entry")
        raw = (CStepEntry * n).from_address(entries_addr)
        entries = [StepEntry(("step", int(e.request)), _ints(e.tokens, e.n_tokens), _ints(e.want, e.n_want)) for e in raw]
        rows = sum(len(e.want) for e in entries)
        if rows > capacity:
            raise ValueError(f"{rows} rows of logits are wanted and logits_out has room for {capacity}")
        if rows and not logits_addr:
            raise ValueError("logits are wanted and logits_out is null")
        logits = self.engine.step(entries)
        if rows:
            host = logits.float().contiguous().cpu()
            C.memmove(logits_addr, host.data_ptr(), host.numel() * 4)
        return rows

    # -- scheduler
    def add(self, rid: int, prompt_addr: int, n: int, params_addr: int) -> None:
        from .engine.scheduler import Request
        if rid in self.requests and self.requests[rid].status != "finished":
            raise ValueError(f"request {rid} is still live")
        req = Request(("sched", rid), _ints(prompt_addr, n), _params(params_addr))
        self.requests[rid] = req
        self.sched.add(req)

    def abort(self, rid: int) -> None:
        if rid not in self.requests:
            raise KeyError(f"no request {rid}")
        self.sched.abort(("sched", rid))

    def sched_step(self, events_addr: int, capacity: int) -> tuple:
        """(number of events written, requests unfinished afterwards)."""
        drawn = {}
        done = self.loop.step()
        if done is not None:
            drawn = done[1]
        events = [(rid[1], tok, 0) for rid, tok in drawn.items()]
        fresh = self.sched.finished[self.reported:]
        self.reported = len(self.sched.finished)
        for req in fresh:
            code = FINISH_CODES.get(req.finish_reason, FINISH_REJECTED)
            for i, (rid, tok, _) in enumerate(events):
                if rid == req.id[1]:
                    events[i] = (rid, tok, code)
                    break
            else:
                events.append((req.id[1], -1, code))
        if len(events) > capacity:
            raise ValueError(f"{len(events)} events and room for {capacity}: give at least max_requests + "
                             "the number of requests added since the last step")
        if events:
            out = (CEvent * len(events)).from_address(events_addr)
            for o, (rid, tok, fin) in zip(out, events):
                o.request, o.token, o.finished = rid, tok, fin
        if not self.sched.has_unfinished() and self.loop.under_way is not None:
            self.loop.step()              # a step started ahead for requests that have all finished since
        return len(events), len(self.sched.waiting) + len(self.sched.running)

    def generate(self, prompt_addr: int, n: int, params_addr: int, out_addr: int, capacity: int) -> int:
        if self.sched.has_unfinished() or self.loop.under_way is not None:
            raise RuntimeError("tuff_generate while requests of tuff_request_add are unfinished")
        gen = self.llm.generate([_ints(prompt_addr, n)], _params(params_addr))[0]
        if gen.finish_reason.startswith("rejected") or gen.finish_reason == "capacity":
            raise ValueError(f"the request was not run: {gen.finish_reason}")
        toks = gen.token_ids[:max(capacity, 0)]
        if toks:
            (C.c_int32 * len(toks)).from_address(out_addr)[:] = toks
        return len(toks)


_sessions: dict = {}
_handles = itertools.count(1)


def open_engine(model_dir: str, dtype: str, max_requests: int, ctx_size: int) -> int:
    h = next(_handles)
    _sessions[h] = Session(model_dir, dtype, max_requests, ctx_size)
    return h


def close_engine(h: int) -> None:
    s = _sessions.pop(h, None)
    if s is not None:
        import gc
        import torch
        del s
        gc.collect()
        torch.cuda.empty_cache()


def session(h: int) -> Session:
    try:
        return _sessions[h]
    except KeyError:
        raise ValueError("the engine handle is closed or was never opened") from None


def info(h: int, what: str) -> int:
    s = session(h)
    if what == "vocab_size":
        return int(s.engine.model.vocab_size)
    if what == "ctx_size":
        return int(s.llm.ctx_size or 0)
    if what == "eos_token":
        eos = s.engine.model.eos_token_id
        return -1 if eos is None else int(eos)
    raise KeyError(what)


def request_begin(h: int, rid: int) -> None:
    session(h).engine.begin(("step", rid))


def request_end(h: int, rid: int) -> None:
    session(h).engine.end(("step", rid))


def request_length(h: int, rid: int) -> int:
    return int(session(h).engine.length(("step", rid)))


def engine_step(h: int, entries_addr: int, n: int, logits_addr: int, capacity: int) -> int:
    return session(h).step(entries_addr, n, logits_addr, capacity)


def request_add(h: int, rid: int, prompt_addr: int, n: int, params_addr: int) -> None:
    session(h).add(rid, prompt_addr, n, params_addr)


def request_abort(h: int, rid: int) -> None:
    session(h).abort(rid)


def sched_step(h: int, events_addr: int, capacity: int) -> tuple:
    return session(h).sched_step(events_addr, capacity)


def generate(h: int, prompt_addr: int, n: int, params_addr: int, out_addr: int, capacity: int) -> int:
    return session(h).generate(prompt_addr, n, params_addr, out_addr, capacity)


def write_random(config_json: str, seed: int, out_dir: str, stored_dtype: str) -> None:
    import torch
    from .models.registry import config_from_dict
    from .weights.random_init import write_random_model
    dtypes = {"bfloat16": torch.bfloat16, "float32": torch.float32}
    if stored_dtype not in dtypes:
        raise ValueError(f"stored_dtype '{stored_dtype}': bfloat16 or float32")
    with open(config_json) as f:
        cfg = config_from_dict(json.load(f))
    write_random_model(cfg, out_dir, int(seed), dtypes[stored_dtype])
