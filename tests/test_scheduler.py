"""The scheduler's decisions (CPU), against a fake step function that checks what it is fed."""
import hashlib

import pytest

from tuff_amd.cache.manager import CacheLayout, CacheManager
from tuff_amd.engine.scheduler import PLACEHOLDER, Request, Scheduler
from tuff_amd.parts.base import FixedState, PagedKV
from tuff_amd.sampling.params import SamplingParams

V = 1000


def next_token(history) -> int:
    """A stand-in model: the next token is a hash of everything before it."""
    return int.from_bytes(hashlib.sha256(repr(list(history)).encode()).digest()[:4], "little") % V


class FakeExecutor:
    """Holds a real CacheManager; 'runs' a step by extending it and checks that every request is
    fed its tokens in order, from the position its cache holds."""

    def __init__(self, num_pages=64, page_size=4, num_slots=4, window=None):
        lay = CacheLayout.from_specs({0: PagedKV(1, 8, window), 1: FixedState((2, 4))})
        self.manager = CacheManager(lay, page_size, num_pages, num_slots)
        self.fed = {}
        self.begun = 0

    def begin(self, rid):
        self.manager.admit(rid)
        self.fed[rid] = []
        self.begun += 1

    def end(self, rid):
        self.manager.release(rid)
        del self.fed[rid]

    def step(self, batch):
        out = {}
        for s in batch:
            rid = s.request.id
            assert s.start == len(self.fed[rid]) == self.manager.length(rid), "fed out of order"
            self.manager.extend(rid, len(s.tokens))         # must never fail: the scheduler promised
            self.fed[rid] += list(s.tokens)
            if s.samples:
                out[rid] = next_token(self.fed[rid])
        self.manager.check()
        return out


def run(sched, ex, max_steps=10000):
    steps = []
    while sched.has_unfinished():
        batch = sched.schedule()
        assert batch, "the scheduler stalled"
        assert sum(len(s.tokens) for s in batch) <= sched.max_batched_tokens
        assert len({s.request.id for s in batch}) == len(batch)
        sched.update(batch, ex.step(batch))
        steps.append(batch)
        assert len(steps) < max_steps
    return steps


def make(ex, **kw):
    kw.setdefault("max_num_seqs", 4)
    kw.setdefault("max_batched_tokens", 16)
    return Scheduler(ex.manager, begin=ex.begin, end=ex.end, **kw)


def expected_output(prompt, n):
    hist, out = list(prompt), []
    for _ in range(n):
        t = next_token(hist)
        out.append(t)
        hist.append(t)
    return out


def test_one_request_prompt_in_portions_then_decode():
    ex = FakeExecutor()
    sched = make(ex, max_batched_tokens=8)
    req = Request("a", list(range(21)), SamplingParams(max_new_tokens=5))
    sched.add(req)
    steps = run(sched, ex)
    assert [len(b[0].tokens) for b in steps] == [8, 8, 5, 1, 1, 1, 1]       # cut under the budget
    assert [b[0].samples for b in steps] == [False, False, True, True, True, True, True]
    assert req.output == expected_output(range(21), 5) and req.finish_reason == "length"
    assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 64


def test_decodes_go_first_and_prompts_share_the_rest_of_the_budget():
    ex = FakeExecutor()
    sched = make(ex, max_batched_tokens=10)
    a = Request("a", list(range(4)), SamplingParams(max_new_tokens=6))
    b = Request("b", list(range(100, 125)), SamplingParams(max_new_tokens=2))
    sched.add(a)
    sched.add(b)
    first = sched.schedule()
    assert [(s.request.id, len(s.tokens)) for s in first] == [("a", 4), ("b", 6)]
    sched.update(first, ex.step(first))
    second = sched.schedule()
    assert [(s.request.id, len(s.tokens), s.samples) for s in second] == [("a", 1, True), ("b", 9, False)]
    sched.update(second, ex.step(second))
    run(sched, ex)
    assert a.output == expected_output(range(4), 6) and b.output == expected_output(range(100, 125), 2)


def test_admission_is_fifo_and_bounded_by_slots_and_max_num_seqs():
    ex = FakeExecutor(num_slots=2)
    sched = make(ex, max_num_seqs=3, max_batched_tokens=64)
    reqs = [Request(i, [i] * 3, SamplingParams(max_new_tokens=3)) for i in range(5)]
    for r in reqs:
        sched.add(r)
    first = sched.schedule()
    assert [s.request.id for s in first] == [0, 1]                       # two slots only
    sched.update(first, ex.step(first))
    steps = run(sched, ex)
    order = []
    for b in [first] + steps:
        for s in b:
            if s.start == 0 and s.request.id not in order:
                order.append(s.request.id)
    assert order == [0, 1, 2, 3, 4]
    assert all(r.output == expected_output([r.id] * 3, 3) for r in reqs)


def test_finish_reasons():
    ex = FakeExecutor()
    sched = make(ex, max_model_len=12, eos_token_id=next_token([5, 6, 7]))
    stop = Request("stop", [5, 6, 7], SamplingParams(max_new_tokens=5))
    ignore = Request("ignore", [5, 6, 7], SamplingParams(max_new_tokens=2, ignore_eos=True))
    too_long = Request("long", list(range(10)), SamplingParams(max_new_tokens=3))
    ctx = Request("ctx", list(range(10)), SamplingParams(max_new_tokens=2))
    zero = Request("zero", [1], SamplingParams(max_new_tokens=0))
    for r in (stop, ignore, too_long, ctx, zero):
        sched.add(r)
    run(sched, ex)
    assert stop.finish_reason == "stop" and len(stop.output) == 1
    assert ignore.finish_reason == "length" and len(ignore.output) == 2
    assert too_long.finish_reason.startswith("rejected") and too_long.output == []
    assert ctx.finish_reason in ("length", "context") and len(ctx.output) == 2
    assert zero.finish_reason == "length" and zero.output == []
    with pytest.raises(ValueError, match="empty prompt"):
        sched.add(Request("e", [], SamplingParams()))


def test_pages_run_out_preempt_the_latest_and_recompute_with_unchanged_output():
    """Pool of 12 pages of 4 tokens; three requests that each grow to 28 tokens (7 pages) cannot
    all stay: the most recently admitted running request is preempted, comes back later and is
    computed again from its first token.  Every output equals the unconstrained one."""
    prompts = {"a": list(range(8)), "b": list(range(50, 58)), "c": list(range(90, 98))}
    ex = FakeExecutor(num_pages=12, page_size=4)
    sched = make(ex, max_batched_tokens=32)
    reqs = {k: Request(k, p, SamplingParams(max_new_tokens=20)) for k, p in prompts.items()}
    for r in reqs.values():
        sched.add(r)
    steps = run(sched, ex)
    assert sched.num_preemptions >= 1
    assert reqs["c"].preemptions >= 1 and reqs["a"].preemptions == 0      # the latest admitted goes first
    for k, p in prompts.items():
        assert reqs[k].output == expected_output(p, 20), k
        assert reqs[k].finish_reason == "length"
    # a preempted request restarts at position 0 with prompt and generated tokens together
    restarts = [s for b in steps for s in b if s.request.id == "c" and s.start == 0]
    assert len(restarts) >= 2
    fed_c = sum(len(s.tokens) for b in steps for s in b if s.request.id == "c")
    assert fed_c > len(prompts["c"]) + 19                                   # tokens were computed again
    after = [s for b in steps[[i for i, b in enumerate(steps) if restarts[-1] in b][0]:] for s in b if s.request.id == "c"]
    assert [s.start for s in after] == [sum(len(x.tokens) for x in after[:i]) for i in range(len(after))]
    assert any(s.start < len(prompts["c"]) < s.start + len(s.tokens) and not s.samples or
               (s.start + len(s.tokens) > len(prompts["c"]) and len(s.tokens) > 1) for s in after)
    assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 12


def test_a_long_prompt_beside_decoding_requests_on_a_tight_pool_is_not_computed_over_and_over():
    """Three requests decode; a fourth with a long prompt is admitted when its first portion fits and
    then finds no pages for the next.  It must wait with what it holds (or take a shorter portion),
    not be preempted and admitted again step after step: tokens computed twice and preemptions stay
    small, and every output is the unconstrained one."""
    prompts = {"a": list(range(6)), "b": list(range(50, 56)), "c": list(range(90, 96)), "long": list(range(200, 260))}
    new = {"a": 22, "b": 18, "c": 14, "long": 4}
    ex = FakeExecutor(num_pages=26, page_size=4)             # 3 x 7 pages at the end of a, b, c; long needs 16
    sched = make(ex, max_batched_tokens=16)
    reqs = {k: Request(k, prompts[k], SamplingParams(max_new_tokens=new[k])) for k in prompts}
    for k in ("a", "b", "c", "long"):
        sched.add(reqs[k])
    steps = run(sched, ex)
    for k in prompts:
        assert reqs[k].output == expected_output(prompts[k], new[k]) and reqs[k].finish_reason == "length", k
    fed = {k: sum(len(s.tokens) for b in steps for s in b if s.request.id == k) for k in prompts}
    needed = {k: len(prompts[k]) + new[k] - 1 for k in prompts}
    assert all(reqs[k].preemptions == 0 and fed[k] == needed[k] for k in ("a", "b", "c"))
    assert sched.num_preemptions <= 2, sched.num_preemptions
    assert reqs["long"].preemptions == sched.num_preemptions
    assert fed["long"] <= needed["long"] * (1 + reqs["long"].preemptions), fed   # at most once over per preemption
    # while it waited for pages it kept the ones it had: steps in which it was left out or got a shorter portion
    waits = [b for b in steps if not any(s.request.id == "long" for s in b) and reqs["long"] in [s.request for bb in steps[:steps.index(b)] for s in bb]]
    short = [s for b in steps for s in b if s.request.id == "long" and not s.samples and len(s.tokens) < 16 - (len(b) - 1)]
    assert waits or short
    assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 26


def test_prompts_that_hold_all_pages_between_them_do_not_stall():
    """Two prompts admitted side by side whose rest fits only one at a time: nothing can move, so
    the later one is preempted and the first goes on."""
    ex = FakeExecutor(num_pages=10, page_size=4)
    sched = make(ex, max_batched_tokens=16)
    a = Request("a", list(range(30)), SamplingParams(max_new_tokens=3))       # 9 pages at the end
    b = Request("b", list(range(100, 130)), SamplingParams(max_new_tokens=3))
    sched.add(a)
    first = sched.schedule()
    sched.update(first, ex.step(first))                                       # a holds 4 pages
    sched.add(b)
    run(sched, ex)
    assert a.output == expected_output(range(30), 3) and b.output == expected_output(range(100, 130), 3)
    assert a.preemptions == 0 and b.preemptions <= 1
    assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 10


def test_decoding_requests_take_turns_when_the_budget_is_smaller_than_their_number():
    ex = FakeExecutor()
    sched = make(ex, max_batched_tokens=4, max_num_seqs=4)
    reqs = [Request(k, [i, i + 1], SamplingParams(max_new_tokens=9)) for i, k in enumerate("abcd")]
    for r in reqs:
        sched.add(r)
    while any(r.remaining() != 1 or r.status != "running" for r in reqs):     # all four decoding
        batch = sched.schedule()
        sched.update(batch, ex.step(batch))
    sched.max_batched_tokens = 3
    seen = []
    for _ in range(4):
        batch = sched.schedule()
        assert len(batch) == 3
        seen.append({s.request.id for s in batch})
        sched.update(batch, ex.step(batch))
    counts = {k: sum(k in b for b in seen) for k in "abcd"}
    assert set(counts.values()) == {3}, counts                               # 12 tokens, three each: nobody starves
    sched.max_batched_tokens = 4
    run(sched, ex)
    for i, r in enumerate(reqs):
        assert r.output == expected_output([i, i + 1], 9)


def test_decoding_requests_take_turns_also_when_every_step_is_decided_ahead():
    """The serving loop decides step k+1 between advance() and commit() of step k, always with ahead=True: the
    turn must move on there too, or the same requests run every step and the others starve until those end."""
    ex = AheadExecutor(num_pages=256, page_size=1)                            # every token needs a page
    sched = make(ex, max_batched_tokens=4, max_num_seqs=4)
    reqs = [Request(k, [i, i + 1], SamplingParams(max_new_tokens=40)) for i, k in enumerate("abcd")]
    for r in reqs:
        sched.add(r)
    while any(r.remaining() != 1 or r.status != "running" for r in reqs):     # all four decoding
        batch = sched.schedule()
        sched.update(batch, ex.step(batch))
    sched.max_batched_tokens = 2
    before = {r.id: len(r.output) for r in reqs}
    batch = sched.schedule()
    sampled = ex.step(batch)
    seen = [{s.request.id for s in batch}]
    for _ in range(7):                                                        # seven more steps, each decided ahead
        sched.advance(batch)
        nxt = sched.schedule(ahead=True)
        assert nxt and len(nxt) == 2
        for s in nxt:
            if PLACEHOLDER in s.tokens:
                s.tokens = [sampled[s.request.id]]
        nxt_sampled = ex.step(nxt)
        sched.commit(batch, sampled)
        seen.append({s.request.id for s in nxt})
        batch, sampled = nxt, nxt_sampled
    sched.advance(batch)
    sched.commit(batch, sampled)
    counts = {k: sum(k in b for b in seen) for k in "abcd"}
    assert set(counts.values()) == {4}, counts                               # 16 tokens, four each
    assert {r.id: len(r.output) - before[r.id] for r in reqs} == {k: 4 for k in "abcd"}
    # a refused ahead call leaves the turn where it was
    turn = sched._decode_turn
    pool = ex.manager.groups[0].pool
    pool._free, kept = [], pool._free                                        # no page left: the call is refused
    assert sched.schedule(ahead=True) is None and sched._decode_turn == turn
    pool._free = kept
    sched.max_batched_tokens = 4
    run(sched, ex)
    for i, r in enumerate(reqs):
        assert r.output == expected_output([i, i + 1], 40)


def test_waiting_request_is_not_admitted_into_a_full_pool():
    ex = FakeExecutor(num_pages=6, page_size=4)
    sched = make(ex, max_batched_tokens=64)
    a = Request("a", list(range(20)), SamplingParams(max_new_tokens=3))      # 5 pages, 6 at the end
    b = Request("b", list(range(8)), SamplingParams(max_new_tokens=2))
    sched.add(a)
    sched.add(b)
    first = sched.schedule()
    assert [s.request.id for s in first] == ["a"]                          # b would not fit beside a
    sched.update(first, ex.step(first))
    run(sched, ex)
    assert a.output == expected_output(range(20), 3) and b.output == expected_output(range(8), 2)
    assert b.preemptions == 0


def test_request_larger_than_the_pool_is_finished_with_capacity():
    ex = FakeExecutor(num_pages=4, page_size=4)
    sched = make(ex)
    big = Request("big", list(range(30)), SamplingParams(max_new_tokens=4))
    ok = Request("ok", list(range(6)), SamplingParams(max_new_tokens=4))
    sched.add(big)
    sched.add(ok)
    run(sched, ex)
    assert big.finish_reason == "capacity" and big.output == []
    assert ok.output == expected_output(range(6), 4)
    assert ex.manager.live() == []


def test_sliding_window_group_needs_fewer_pages():
    """With a window of 8 a request of 60 tokens runs in a pool of 5 pages of 4."""
    ex = FakeExecutor(num_pages=5, page_size=4, window=8)
    sched = make(ex, max_batched_tokens=4)
    r = Request("w", list(range(40)), SamplingParams(max_new_tokens=20))
    sched.add(r)
    run(sched, ex)
    assert r.output == expected_output(range(40), 20) and r.preemptions == 0
    assert ex.manager.groups[0].pool.allocations > 5


def test_abort_gives_everything_back():
    ex = FakeExecutor()
    sched = make(ex)
    a = Request("a", list(range(10)), SamplingParams(max_new_tokens=50))
    b = Request("b", list(range(10)), SamplingParams(max_new_tokens=50))
    sched.add(a)
    sched.add(b)
    for _ in range(3):
        batch = sched.schedule()
        sched.update(batch, ex.step(batch))
    sched.abort("a")
    assert a.finish_reason == "aborted" and ex.manager.live() == ["b"]
    sched.abort("b")
    assert not sched.has_unfinished() and ex.manager.groups[0].pool.num_free == 64 and ex.manager.free_slots == 4


def test_seeded_sampling_state_survives_preemption():
    """The per-request generator is not reset by a preemption: draws continue where they were."""
    from tuff_amd.sampling.params import SamplerState
    p = SamplingParams(temp=0.8, seed=11, max_new_tokens=4)
    r = Request("x", [1, 2], p)
    ex = FakeExecutor()
    sched = make(ex)
    sched.add(r)
    first = [r.sampler.rng.uniform() for _ in range(2)]
    fresh = SamplerState(p)
    assert first == [fresh.rng.uniform() for _ in range(2)]
    nxt = fresh.rng.uniform()
    sched.running.append(sched.waiting.popleft())
    ex.begin("x")
    sched._preempt(r)
    assert r.sampler.rng.uniform() == nxt and r.num_computed == 0 and sched.waiting[0] is r


# ---------------------------------------------------------------- deciding a step ahead
def run_ahead(sched, ex, stats=None):
    """The loop of LLM.run over the fake executor: the next step is decided between advance() and
    commit() and 'started' (the executor extends the cache) before the current step's tokens are
    handed over; the executor sees the real token where the scheduler has a placeholder, as the
    GPU does."""
    steps, ahead = [], 0
    under_way = None
    while under_way is not None or sched.has_unfinished():
        if under_way is None:
            batch = sched.schedule()
            assert batch, "the scheduler stalled"
            sampled = ex.step(batch)
        else:
            batch, sampled = under_way
            under_way = None
        live = sched.advance(batch)
        nxt = sched.schedule(ahead=True)
        if nxt:
            assert sum(len(s.tokens) for s in nxt) <= sched.max_batched_tokens
            assert len({s.request.id for s in nxt}) == len(nxt)
            for s in nxt:
                if PLACEHOLDER in s.tokens:
                    assert len(s.tokens) == 1 and s.samples
                    s.tokens = [sampled[s.request.id]]
            under_way = (nxt, ex.step(nxt))
            ahead += 1
            if stats is not None and any(len(s.tokens) > 1 for s in nxt):
                stats["mixed"] = stats.get("mixed", 0) + 1
        sched.commit(batch, sampled)
        for r in list(sched.running) + list(sched.waiting) + sched.finished:
            assert PLACEHOLDER not in r.output
        steps.append(live)
    return steps, ahead


class AheadExecutor(FakeExecutor):
    """A request may end (and be released) while a step that holds it is under way."""

    def end(self, rid):
        self.manager.release(rid)
        self.fed.pop(rid, None)


def test_a_step_decided_ahead_feeds_the_same_tokens():
    prompts = {"a": list(range(9)), "b": list(range(40, 47)), "c": list(range(100, 103)), "d": list(range(200, 231)),
               "e": list(range(300, 305))}
    new = {"a": 12, "b": 7, "c": 20, "d": 3, "e": 1}
    outs = {}
    for mode in ("plain", "ahead"):
        ex = AheadExecutor()
        sched = make(ex, max_batched_tokens=8, max_num_seqs=3)
        reqs = {k: Request(k, prompts[k], SamplingParams(max_new_tokens=new[k])) for k in prompts}
        for r in reqs.values():
            sched.add(r)
        if mode == "plain":
            run(sched, ex)
        else:
            stats = {}
            steps, ahead = run_ahead(sched, ex, stats)
            assert ahead == len(steps) - 1 and stats["mixed"] >= 4      # portions of prompts too
        outs[mode] = {k: r.output for k, r in reqs.items()}
        assert all(r.finish_reason == "length" for r in reqs.values())
        assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 64
    assert outs["plain"] == outs["ahead"]
    assert outs["plain"]["a"] == expected_output(prompts["a"], 12)


def test_a_step_ahead_holds_placeholders_and_leaves_out_who_is_sure_to_end():
    ex = AheadExecutor()
    sched = make(ex, max_batched_tokens=8)
    a = Request("a", list(range(7)), SamplingParams(max_new_tokens=2))
    b = Request("b", list(range(20, 26)), SamplingParams(max_new_tokens=30))
    sched.add(a)
    batch = sched.schedule()                      # a's prompt: 7 tokens, samples
    sampled = ex.step(batch)
    sched.add(b)
    assert sched.advance(batch) == batch and a.output == [PLACEHOLDER] and a.num_computed == 7
    nxt = sched.schedule(ahead=True)              # a decodes the token nobody has seen, b is admitted beside it
    assert [(s.request.id, s.start, s.tokens, s.samples) for s in nxt] == \
        [("a", 7, [PLACEHOLDER], True), ("b", 0, list(range(20, 26)), True)]
    nxt[0].tokens = [sampled["a"]]
    sampled2 = ex.step(nxt)
    assert sched.commit(batch, sampled) == [] and a.output == [sampled["a"]]
    sched.advance(nxt)                            # a's second token is its last: it gives back what it holds now
    assert a.status == "finished" and a not in sched.running and ex.manager.live() == ["b"]
    assert a not in sched.finished and a.output[1] == PLACEHOLDER
    third = sched.schedule(ahead=True)
    assert [(s.request.id, s.tokens) for s in third] == [("b", [PLACEHOLDER])]
    assert sched.commit(nxt, sampled2) == [a] and a.finish_reason == "length" and sched.finished == [a]
    assert a.output == expected_output(range(7), 2)


def test_deciding_ahead_stops_where_pages_run_out():
    """Three pages of four tokens for two requests that need two each: when both want their second
    page no step is decided ahead (and nothing is changed by the attempt), schedule() preempts,
    and the output is what it would have been."""
    outs = {}
    for mode in ("plain", "ahead"):
        ex = AheadExecutor(num_pages=3)
        sched = make(ex)
        reqs = [Request(k, list(range(i, i + 3)), SamplingParams(max_new_tokens=4)) for i, k in enumerate("ab")]
        for r in reqs:
            sched.add(r)
        if mode == "plain":
            run(sched, ex)
        else:
            steps, ahead = run_ahead(sched, ex)
            assert ahead < len(steps) - 1
        assert sched.num_preemptions >= 1
        outs[mode] = [r.output for r in reqs]
        assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 3
    assert outs["plain"] == outs["ahead"] == [expected_output(range(i, i + 3), 4) for i in range(2)]


def test_a_request_that_ends_while_the_next_step_is_under_way():
    ex = AheadExecutor()
    sched = make(ex, eos_token_id=None)
    a = Request("a", list(range(5)), SamplingParams(max_new_tokens=30))
    b = Request("b", list(range(50, 58)), SamplingParams(max_new_tokens=30))
    sched.add(a)
    sched.add(b)
    free_run_a = expected_output(range(5), 30)
    sched.eos_token_id = free_run_a[6]            # a stops after its 7th token
    steps, ahead = run_ahead(sched, ex)
    cut = free_run_a.index(free_run_a[6]) + 1
    assert a.output == free_run_a[:cut] and a.finish_reason == "stop"
    assert len(b.output) <= 30 and b.finish_reason in ("length", "stop")
    want_b = expected_output(range(50, 58), 30)
    assert b.output == want_b[:len(b.output)]
    assert all(s.request is not a for live in steps[cut + 1:] for s in live)   # the step under way did not count
    assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 64
    ex.manager.check()


@pytest.mark.parametrize("seed", range(12))
def test_random_scenarios_ahead_equal_plain(seed):
    """Requests of random lengths over a small pool, with a window group or without, with an
    end-of-sequence token that some of them hit: the loop that starts steps early produces what the
    plain loop produces, and gives everything back."""
    import random
    rng = random.Random(seed)
    pages, window = rng.choice([6, 10, 24]), rng.choice([None, 8])
    budget, seqs = rng.choice([4, 7, 16]), rng.choice([1, 2, 4])
    spec = [(list(range(100 * i, 100 * i + rng.randrange(1, 14))), rng.randrange(1, 10)) for i in range(rng.randrange(2, 9))]
    eos = next_token(spec[0][0]) if rng.random() < 0.5 else None
    outs = {}
    for mode in ("plain", "ahead"):
        ex = AheadExecutor(num_pages=pages, window=window)
        sched = make(ex, max_batched_tokens=budget, max_num_seqs=seqs, eos_token_id=eos)
        reqs = [Request(i, p, SamplingParams(max_new_tokens=n)) for i, (p, n) in enumerate(spec)]
        for r in reqs:
            sched.add(r)
        (run if mode == "plain" else run_ahead)(sched, ex)
        outs[mode] = [(r.output, r.finish_reason) for r in reqs]
        assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == pages and ex.manager.free_slots == 4
        assert sorted(r.id for r in sched.finished) == list(range(len(spec)))
    assert outs["plain"] == outs["ahead"]


# ------------------------------------------------------- a step that fails midway
class _Out:
    """Stands in for the sampler's output tensor on the device."""

    def __init__(self, values):
        self.values, self.shape = list(values), (len(values),)


class _Pending:
    def __init__(self, values):
        self.out = _Out(values)

    def tokens(self):
        return list(self.out.values)


class _FakeSampler:
    def launch(self, logits, samplers):
        assert len(logits) == len(samplers)
        return _Pending(logits)

    def needs_history(self, sampler):
        return False


class _FakeEngine:
    """Engine.step over the fake executor: resolves tokens that are still 'on the device', checks the order of
    what it is fed, and fails midway at the call it is told to, as a refused launch would."""

    def __init__(self, ex, fail_at_call):
        self.ex, self.fail_at_call, self.calls = ex, fail_at_call, 0

    def step(self, entries, device_tokens=None):
        from tuff_amd.engine.engine import StepFailed
        self.calls += 1
        flat = [t for e in entries for t in e.tokens]
        if device_tokens is not None:
            if isinstance(device_tokens, _Out):
                flat = list(device_tokens.values)
            else:
                out, places, sources = device_tokens
                for p, q in zip(places, sources):
                    flat[p] = out.values[q]
        if self.calls == self.fail_at_call:
            raise StepFailed([e.req_id for e in entries], RuntimeError("launch refused")) from RuntimeError("launch refused")
        logits, at = [], 0
        for e in entries:
            toks = flat[at:at + len(e.tokens)]
            at += len(e.tokens)
            assert self.ex.manager.length(e.req_id) == len(self.ex.fed[e.req_id])
            self.ex.manager.extend(e.req_id, len(toks))
            self.ex.fed[e.req_id] += toks
            for _ in e.want:
                logits.append(next_token(self.ex.fed[e.req_id]))
        self.ex.manager.check()
        return logits


@pytest.mark.parametrize("run_ahead", [True, False])
@pytest.mark.parametrize("fail_at_call", [1, 2, 4, 7])
def test_the_run_loop_ends_the_requests_of_a_step_that_failed_midway(fail_at_call, run_ahead):
    """Engine.step raises StepFailed after some kernels ran: what the step's requests hold is gone.  The loop ends
    exactly those requests with the reason, their pages and slots come back, nothing that was drawn and not yet
    seen is left in their output, and the other requests go on to the right tokens when the loop is called again."""
    import types
    from tuff_amd.engine.engine import StepFailed
    from tuff_amd.engine.llm import Loop
    ex = AheadExecutor(num_pages=64, page_size=4)
    sched = make(ex, max_batched_tokens=3, max_num_seqs=4)                    # no step holds all four requests
    reqs = [Request(k, [i, i + 1, i + 2], SamplingParams(max_new_tokens=6)) for i, k in enumerate("abcd")]
    for r in reqs:
        sched.add(r)
    llm = types.SimpleNamespace(engine=_FakeEngine(ex, fail_at_call), sampler=_FakeSampler(), run_ahead=run_ahead)
    loop = Loop(llm, sched)
    failures = []
    for _ in range(200):
        try:
            if loop.step() is None:
                break
        except StepFailed as e:
            failures.append(e)
    assert len(failures) == 1 and not sched.has_unfinished()
    hit = set(failures[0].requests)
    assert hit and hit < set("abcd")
    for i, r in enumerate(reqs):
        assert r.status == "finished" and PLACEHOLDER not in r.output
        if r.id in hit:
            assert r.finish_reason.startswith("error: launch refused")
            assert r.output == expected_output([i, i + 1, i + 2], 6)[:len(r.output)]       # what it got before is right
        else:
            assert r.finish_reason == "length" and r.output == expected_output([i, i + 1, i + 2], 6)
    ex.manager.check()
    assert ex.manager.live() == [] and ex.manager.groups[0].pool.num_free == 64


@pytest.mark.parametrize("run_ahead", [True, False])
@pytest.mark.parametrize("num_pages", [64, 9])
def test_the_run_loop_brings_what_comes_with_the_tokens_for_the_places_it_feeds(run_ahead, num_pages):
    """Requests whose tokens come with more than their ids (Request.inputs, a function of the place): every entry
    of every step holds the inputs of exactly the places it feeds, for prompt portions, for tokens that are not
    drawn yet when the step is decided, and for the tokens fed again after a preemption (the small pool)."""
    import types
    from tuff_amd.engine.llm import Loop
    ex = AheadExecutor(num_pages=num_pages, page_size=4)
    seen = []

    class Engine(_FakeEngine):
        def step(self, entries, device_tokens=None):
            for e in entries:
                at = self.ex.manager.length(e.req_id)
                assert e.inputs is not None and list(e.inputs["place"]) == [[at + i, 100 * int(e.req_id)] for i in range(len(e.tokens))]
                seen.append((e.req_id, at, len(e.tokens)))
            return super().step(entries, device_tokens)

    sched = make(ex, max_batched_tokens=5, max_num_seqs=3)
    reqs = [Request(k, list(range(10 * k, 10 * k + n)), SamplingParams(max_new_tokens=new),
                    inputs=lambda start, n, k=k: {"place": [[start + i, 100 * k] for i in range(n)]})
            for k, (n, new) in enumerate([(7, 9), (3, 12), (11, 4), (2, 8)])]
    for r in reqs:
        sched.add(r)
    llm = types.SimpleNamespace(engine=Engine(ex, fail_at_call=-1), sampler=_FakeSampler(), run_ahead=run_ahead)
    loop = Loop(llm, sched)
    for _ in range(500):
        if loop.step() is None:
            break
    assert not sched.has_unfinished()
    for k, r in enumerate(reqs):
        assert r.finish_reason == "length" and r.output == expected_output(r.prompt, r.params.max_new_tokens)
    if num_pages == 9:
        assert sum(r.preemptions for r in reqs) >= 1
        assert any(at == 0 and rid == r.id for r in reqs if r.preemptions for rid, at, n in seen[1:])
    assert any(n > 1 for _, _, n in seen) and any(n == 1 for _, _, n in seen)
    ex.manager.check()
    assert ex.manager.live() == []
