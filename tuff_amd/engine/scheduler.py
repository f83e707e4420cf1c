"""Continuous batching above the step function.

Every call to `schedule()` decides one step: requests that are decoding get their one token
first, then prompts are continued and new requests admitted, in arrival order, while the
token budget, the state slots and the pages last; the last prompt portion is cut to fit the
budget.  `update()` takes the sampled tokens, finishes requests and frees what they held.  It has
two halves for a caller that starts the next step before it has seen this one's tokens:
`advance()` accounts for a step that has been started (positions move on, every request that draws
a token gets a PLACEHOLDER at the end of its output, requests that end with this token whatever it
is are finished), `commit()` puts the tokens where the placeholders are and finishes requests at
an end-of-sequence token.  Between the two, `schedule(ahead=True)` decides the next step.

When pages run out: a waiting request is simply not admitted yet.  A running prompt whose next
portion does not fit is cut to the pages there are, or sits a step out with what it holds.  If a
decoding request cannot get the page for its next token, the most recently admitted running
request is preempted: its pages and slot are given back, and it returns to the head of the
waiting queue to be computed again from its first token, prompt and generated tokens together (a
conv state cannot be rebuilt from the KV cache, so recomputation is the only exact way); it is not
admitted again in the call that preempted it.  Its sampler state is kept, so its draws do not
change.  A request that does not fit the pool even alone is finished with reason "capacity".

The reference runs one request and has no scheduler; the loop shape follows its other
backend's slot loop (src/qwen35/q35_server.c:869-1050): FIFO admission, prompt portions beside
one decode batch, slot freed at finish.
"""
from __future__ import annotations

import collections
import dataclasses
from typing import Callable, Hashable, Optional

from ..cache.manager import CacheManager
from ..sampling.params import SamplerState, SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"
PLACEHOLDER = -1                 # in Request.output: a token that has been drawn on the device and not yet seen


@dataclasses.dataclass(eq=False)           # a request is itself: lists of requests are searched by identity
class Request:
    id: Hashable
    prompt: list
    params: SamplingParams
    output: list = dataclasses.field(default_factory=list)
    status: str = WAITING
    num_computed: int = 0            # tokens of prompt+output whose cache entries exist
    finish_reason: Optional[str] = None
    preemptions: int = 0
    sampler: Optional[SamplerState] = None
    # inputs(start, n) -> {name: integers [n] or [n, cols]} for the tokens at places start .. start + n - 1 of
    # prompt + output, where the model's parts read more of a token than its id and position (StepEntry.inputs);
    # a function of the place, so that it also answers for tokens that are not drawn yet and after a preemption
    inputs: Optional[Callable] = None

    def tokens(self) -> list:
        return self.prompt + self.output

    def token_slice(self, start: int, n: int) -> list:
        """tokens()[start:start + n] without building the whole list."""
        np_ = len(self.prompt)
        if start >= np_:
            return self.output[start - np_:start - np_ + n]
        if start + n <= np_:
            return self.prompt[start:start + n]
        return self.prompt[start:] + self.output[:start + n - np_]

    def remaining(self) -> int:
        return len(self.prompt) + len(self.output) - self.num_computed


@dataclasses.dataclass
class Scheduled:
    request: Request
    start: int                       # first position fed in this step
    tokens: list
    samples: bool                    # the step reaches the request's last token: draw the next
    counted: bool = True             # advance(): the request was live when the step was accounted
    slot: int = -1                   # advance(): where in Request.output the drawn token goes
    finishes: bool = False           # advance(): the request ends with this token, whatever it is


class Scheduler:
    def __init__(self, manager: CacheManager, *, begin, end, max_num_seqs: int = 8,
                 max_batched_tokens: int = 2048, max_model_len: Optional[int] = None,
                 eos_token_id: Optional[int] = None):
        """begin(req_id) / end(req_id): take and give back a request's cache (Engine.begin/end)."""
        self.manager, self._begin, self._end = manager, begin, end
        self.max_num_seqs = int(max_num_seqs)
        self.max_batched_tokens = int(max_batched_tokens)
        self.max_model_len = max_model_len
        self.eos_token_id = eos_token_id
        if self.max_batched_tokens < 1 or self.max_num_seqs < 1:
            raise ValueError("max_batched_tokens and max_num_seqs must be positive")
        self.waiting: collections.deque[Request] = collections.deque()
        self.running: list[Request] = []          # in admission order
        self.finished: list[Request] = []
        self.num_preemptions = 0
        self._decode_turn = 0                     # where the decoding requests' turns go on (budget < requests)
        self._turn_pending = 0                    # by how much the step being decided moves the turn on

    # ------------------------------------------------------------------- requests
    def add(self, req: Request) -> None:
        req.params.validate()
        if not req.prompt:
            raise ValueError(f"request {req.id!r}: empty prompt")
        if req.sampler is None:
            req.sampler = SamplerState(req.params)
        if self.max_model_len is not None and len(req.prompt) + req.params.max_new_tokens > self.max_model_len:
            # the reference checks the same up front (ctx_fits, src/main.c:687-692, :1264-1275)
            self._finish(req, "rejected: prompt + max_new_tokens exceeds the context length")
            return
        if req.params.max_new_tokens == 0:
            self._finish(req, "length")
            return
        self.waiting.append(req)

    def adopt(self, req: Request, num_computed: int) -> None:
        """Takes over a request that is already live in the cache with its first
        `num_computed` tokens computed (begin() and the steps were done by the caller)."""
        req.params.validate()
        if self.manager.length(req.id) != num_computed or not 0 <= num_computed < len(req.prompt) + len(req.output):
            raise ValueError(f"request {req.id!r}: the cache holds {self.manager.length(req.id)} tokens, "
                             f"not the {num_computed} stated")
        if req.sampler is None:
            req.sampler = SamplerState(req.params)
        req.status, req.num_computed = RUNNING, num_computed
        self.running.append(req)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def abort(self, req_id, reason: str = "aborted") -> None:
        """Ends a request wherever it is and gives back what it holds.  A token that was drawn and not yet seen
        (a PLACEHOLDER at the end of its output) is dropped."""
        for r in list(self.running):
            if r.id == req_id:
                self.running.remove(r)
                self._end(r.id)
                self._drop_placeholders(r)
                self._finish(r, reason)
                return
        for r in list(self.waiting):
            if r.id == req_id:
                self.waiting.remove(r)
                self._drop_placeholders(r)
                self._finish(r, reason)
                return

    @staticmethod
    def _drop_placeholders(req: Request) -> None:
        while req.output and req.output[-1] == PLACEHOLDER:
            req.output.pop()

    def _finish(self, req: Request, reason: str) -> None:
        req.status, req.finish_reason = FINISHED, reason
        self.finished.append(req)

    # ------------------------------------------------------------------- one step
    def _fits(self, req: Request, n: int, promised: list[int]) -> bool:
        need = self.manager.pages_needed(req.id, n)
        back = self.manager.reclaimable(req.id)
        return all(nd <= g.pool.num_free + b - p
                   for nd, b, p, g in zip(need, back, promised, self.manager.groups))

    def _promise(self, req: Request, n: int, promised: list[int]) -> None:
        need = self.manager.pages_needed(req.id, n)
        back = self.manager.reclaimable(req.id)
        for i, (nd, b) in enumerate(zip(need, back)):
            promised[i] += nd - b

    def _preempt(self, victim: Request) -> None:
        self.running.remove(victim)
        self._end(victim.id)
        victim.status, victim.num_computed = WAITING, 0
        victim.preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(victim)

    def _total_pages(self) -> list[int]:
        return [g.pool.num_pages for g in self.manager.groups]

    def _largest_fit(self, req: Request, n: int, promised: list[int]) -> int:
        """The most tokens of `req`, at most n, whose pages are there (0: not even one)."""
        if not self._fits(req, 1, promised):
            return 0
        lo, hi = 1, n                                         # lo fits; pages needed grow with the tokens
        while lo < hi:
            mid = (lo + hi + 1) // 2
            if self._fits(req, mid, promised):
                lo = mid
            else:
                hi = mid - 1
        return lo

    def schedule(self, ahead: bool = False) -> Optional[list[Scheduled]]:
        """The next step.  ahead: the step before has been through advance() and not through
        commit(); tokens not yet seen appear as PLACEHOLDER in Scheduled.tokens (always as the one
        token of a decoding request).  Nobody can be preempted then, since a request's tokens must
        be known to compute it again: where a running request lacks pages the answer is None, and
        nothing has been changed.

        Who yields when pages are short: a prompt portion is cut to the pages there are, or waits a
        step with what it holds; only a decoding request that cannot grow preempts, the most recently
        admitted running request first.  If nothing at all can move (prompts holding all pages
        between them), the most recently admitted one is preempted.  A request preempted in this call
        is not admitted again in it."""
        preempted_now: set[int] = set()
        while True:
            self._turn_pending = 0
            out = self._schedule_once(ahead, preempted_now)
            if out is None or out or not self.running or ahead:
                if out:
                    # the turn moves on when a step is really handed out, also one decided ahead (a serving loop
                    # that always decides ahead would otherwise run the same requests every step); a refused
                    # ahead call (None) changes nothing
                    self._decode_turn += self._turn_pending
                return out
            # running requests and none can take a token: make room
            victim = self.running[-1]
            if len(self.running) == 1:
                self.running.remove(victim)
                self._end(victim.id)
                self._finish(victim, "capacity")
            else:
                self._preempt(victim)
                preempted_now.add(id(victim))

    def _schedule_once(self, ahead: bool, preempted_now: set) -> Optional[list[Scheduled]]:
        budget = self.max_batched_tokens
        promised = [0] * len(self.manager.groups)
        out: list[Scheduled] = []

        # running requests, decoding ones first, then prompts in admission order
        rank = {id(r): i for i, r in enumerate(self.running)}
        order = sorted(self.running, key=lambda r: (r.remaining() != 1, rank[id(r)]))
        n_decoding = sum(1 for r in order if r.remaining() == 1)
        if n_decoding > budget:
            # fewer tokens a step than decoding requests: they take turns, each step going on where
            # the one before stopped
            turn = self._decode_turn % n_decoding
            order = order[turn:n_decoding] + order[:turn] + order[n_decoding:]
            self._turn_pending = budget
        for req in order:
            if req not in self.running or budget == 0:       # preempted meanwhile / nothing left
                continue
            n = min(req.remaining(), budget)
            if not self._fits(req, n, promised):
                if ahead:
                    return None
                if req.remaining() > 1:
                    # a prompt (or a request being computed again): what fits, or nothing this step
                    n = self._largest_fit(req, n, promised)
                else:
                    n = self._make_room_for_a_decoding_request(req, out, promised, preempted_now)
                    budget = self.max_batched_tokens - sum(len(s.tokens) for s in out)
            if n == 0:
                continue
            self._promise(req, n, promised)
            toks = req.token_slice(req.num_computed, n)
            out.append(Scheduled(req, req.num_computed, toks, req.num_computed + n == len(req.prompt) + len(req.output)))
            budget -= n

        # admit waiting requests in order while slots, budget and pages last
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs \
                and self.manager.free_slots > 0:
            req = self.waiting[0]
            if id(req) in preempted_now:
                break
            total = len(req.prompt) + req.params.max_new_tokens
            need_alone = -(-total // self.manager.page_size)
            windows = [g.window for g in self.manager.groups]
            if any(w is None and need_alone > tp for w, tp in zip(windows, self._total_pages())):
                self.waiting.popleft()
                self._finish(req, "capacity")
                continue
            self._begin(req.id)
            n = min(req.remaining(), budget)
            if not self._fits(req, n, promised):
                # a shorter first portion; if not even one token fits, wait
                n = self._largest_fit(req, n, promised)
                if n == 0 or self.running:
                    self._end(req.id)
                    break
            self.waiting.popleft()
            req.status = RUNNING
            self.running.append(req)
            self._promise(req, n, promised)
            toks = req.token_slice(0, n)
            out.append(Scheduled(req, 0, toks, n == len(req.prompt) + len(req.output)))
            budget -= n
        return out

    def _make_room_for_a_decoding_request(self, req: Request, out: list, promised: list[int], preempted_now: set) -> int:
        """Preempts the most recently admitted running requests until req's one token has its page.
        Returns the tokens req gets (1, or 0 if it went itself); `promised` is brought up to date
        in place and entries of preempted requests leave `out`."""
        while not self._fits(req, 1, promised):
            victim = self.running[-1]
            if victim is req and len(self.running) == 1:
                self.running.remove(req)
                self._end(req.id)
                self._finish(req, "capacity")
                return 0
            scheduled_victim = next((s for s in out if s.request is victim), None)
            if scheduled_victim is not None:
                out.remove(scheduled_victim)
                promised[:] = [0] * len(self.manager.groups)
                for s in out:
                    self._promise(s.request, len(s.tokens), promised)
            self._preempt(victim)
            preempted_now.add(id(victim))
            if victim is req:
                return 0
        return 1

    def update(self, scheduled: list[Scheduled], sampled: dict) -> list[Request]:
        """sampled: {request id: token} for every Scheduled with samples=True.
        Returns the requests that finished in this step."""
        self.advance(scheduled)
        return self.commit(scheduled, sampled)

    def advance(self, scheduled: list[Scheduled]) -> list[Scheduled]:
        """Accounts for a step that has been started and whose tokens are not known yet.
        Returns the entries that count: those whose requests had not finished meanwhile (a step
        that was started early may hold a request that ended with the token before)."""
        live = []
        for s in scheduled:
            req = s.request
            s.counted = req.status != FINISHED
            if not s.counted:
                continue
            live.append(s)
            req.num_computed += len(s.tokens)
            if not s.samples:
                continue
            s.slot = len(req.output)
            req.output.append(PLACEHOLDER)
            reason = None
            if len(req.output) >= req.params.max_new_tokens:
                reason = "length"
            elif self.max_model_len is not None and len(req.prompt) + len(req.output) >= self.max_model_len:
                reason = "context"
            if reason:
                # what it holds can go back now: whoever takes it runs after this step
                s.finishes = True
                self.running.remove(req)
                self._end(req.id)
                req.status, req.finish_reason = FINISHED, reason
        return live

    def commit(self, scheduled: list[Scheduled], sampled: dict) -> list[Request]:
        """The tokens of a step that advance() has accounted for.  Returns the requests that
        finished in this step."""
        done = []
        for s in scheduled:
            if not (s.counted and s.samples):
                continue
            req = s.request
            tok = int(sampled[req.id])
            req.output[s.slot] = tok
            stop = self.eos_token_id is not None and tok == self.eos_token_id and not req.params.ignore_eos
            if s.finishes:
                if stop:
                    req.finish_reason = "stop"
                self.finished.append(req)
                done.append(req)
            elif stop and req.status == RUNNING:
                self.running.remove(req)
                self._end(req.id)
                self._finish(req, "stop")
                done.append(req)
        return done
