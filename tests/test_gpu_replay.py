"""The engine against the plain implementation under every way of cutting and batching:
whole requests, a long head then 32 single tokens, portions of changing size, and up to four
live requests mixed with so few pages that they are used again.  float32 and bfloat16."""
import os

import pytest
import torch

import util

pytestmark = pytest.mark.gpu

LENGTHS = [45, 70, 100, 33, 129, 64]


def requests_for(name):
    V = util.CONFIGS[name.rstrip("+")][0]["vocab_size"]
    return {f"r{i}": util.rand_tokens(n, V, 100 * i + len(name)) for i, n in enumerate(LENGTHS)}


def stored_for(dtype):
    return "float32" if dtype == "float32" else "bfloat16"


def make_engine(name, dtype, **kw):
    from tuff_amd.engine.engine import Engine
    kw.setdefault("page_size", 16)
    kw.setdefault("max_tokens", 1024)
    kw.setdefault("poison_cache", True)          # NaN in every page that nobody has written since it was handed out
    return Engine.from_folder(util.model_folder(name, stored_for(dtype)), dtype=dtype, **kw)


def check_plan(name, dtype, plan, reqs, **kw):
    eng = make_engine(name, dtype, **kw)
    got = util.run_plan(eng, plan)
    eng.manager.check()
    assert not eng.manager.live()
    for rid, toks in reqs.items():
        want = util.expected(name, toks, stored_for(dtype))
        util.assert_close(dtype, got[rid], want, f"{name}/{dtype}/{rid}")
    return eng, got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "G"])
def test_whole(gpu, name, dtype):
    reqs = requests_for(name)
    check_plan(name, dtype, util.plan_whole(reqs), reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A+", "B+"])
def test_loud_conv_mixers(gpu, name, dtype):
    """The conv mixers' weights scaled up until they add more than the residual stream holds: a fault in
    the conv state (a wrong slot, a wrong shift, a state that a portion's edge loses) then shows in
    bfloat16 too, where random weights of the usual size would hide it under the rounding."""
    reqs = requests_for(name)
    check_plan(name, dtype, util.plan_tail(reqs, 32), reqs)
    check_plan(name, dtype, util.plan_chunks(reqs, sizes=(2, 3, 2, 29, 5)), reqs)
    plan = util.plan_mixed(reqs, seed=6)
    check_plan(name, dtype, plan, reqs, max_tokens=util.live_tokens_peak(plan), max_requests=4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [16, 48, 64])
def test_heads_of_64_and_other_page_sizes(gpu, page_size, dtype):
    """Heads of 64 channels (the single-token kernels that do norm, rotation, cache write and attention in
    one, and projection and convolution in one, are for them) on pages of 16, 48 and 64 positions:
    a head and single tokens, changing portions, and mixed with pages that are used again."""
    reqs = requests_for("E")
    check_plan("E", dtype, util.plan_tail(reqs, 32), reqs, page_size=page_size)
    check_plan("E", dtype, util.plan_chunks(reqs, sizes=(2, 3, 2, 29, 5)), reqs, page_size=page_size)
    plan = util.plan_mixed(reqs, seed=8)
    peak = -(-util.live_tokens_peak(plan) // page_size) * page_size + 4 * page_size
    check_plan("E", dtype, plan, reqs, page_size=page_size, max_tokens=peak, max_requests=4)


@pytest.mark.parametrize("page_size", [96, 112])
def test_pages_that_do_not_divide_a_partition_of_keys(gpu, page_size):
    """Pages of 96 and 112 positions under a request of 1,200 tokens in bfloat16: the single-token attention cuts
    the keys into partitions of 256, and a partition that starts inside a page touches one page more than
    256 / page size rounded up.  A head in portions, then single tokens across the partition edge at 1,024
    and beyond 1,100, beside a short request."""
    V = util.CONFIGS["E"][0]["vocab_size"]
    reqs = {"long": util.rand_tokens(1200, V, 77), "short": util.rand_tokens(140, V, 78)}
    steps, at = [], {"long": 0, "short": 0}

    def step(parts):
        entries = []
        for rid, n in parts:
            toks = reqs[rid][at[rid]:at[rid] + n]
            at[rid] += len(toks)
            if toks:
                entries.append({"id": rid, "tokens": toks, "want": list(range(len(toks)))})
        steps.append({"step": len(steps), "entries": entries, "end": []})
    step([("long", 500)])
    step([("long", 500), ("short", 100)])
    while at["long"] < 1200:
        step([("long", 1), ("short", 1)])
    steps[-1]["end"] = ["long", "short"]
    check_plan("E", "bfloat16", steps, reqs, page_size=page_size, max_tokens=16 * page_size)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n_req", [("A+", 20), ("E", 37), ("B+", 64)])
def test_many_requests_decode_together(gpu, name, n_req, dtype):
    """17 to 64 requests bring one token each in a step: the products of that many rows, the convolution in
    the kernel that adds their slices, attention over many short requests.  Heads of the prompts in one
    step of portions, then twelve steps of single tokens of all requests."""
    V = util.CONFIGS[name.rstrip("+")][0]["vocab_size"]
    tail = 12
    reqs = {f"r{i}": util.rand_tokens(tail + 2 + (7 * i) % 19, V, 300 + i) for i in range(n_req)}
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:len(toks) - tail], "want": list(range(len(toks) - tail))}
                                     for rid, toks in reqs.items()], "end": []}]
    for j in range(tail):
        steps.append({"step": len(steps), "end": [],
                      "entries": [{"id": rid, "tokens": [toks[len(toks) - tail + j]], "want": [0]} for rid, toks in reqs.items()]})
    steps[-1]["end"] = list(reqs)
    check_plan(name, dtype, steps, reqs, max_tokens=64 * n_req, max_requests=n_req)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_width_that_is_no_multiple_of_8(gpu, dtype):
    reqs = requests_for("D")
    check_plan("D", dtype, util.plan_whole(reqs), reqs)
    plan = util.plan_mixed(reqs, seed=4)
    check_plan("D", dtype, plan, reqs, max_tokens=util.live_tokens_peak(plan))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "G"])
def test_head_then_single_tokens(gpu, name, dtype):
    reqs = requests_for(name)
    check_plan(name, dtype, util.plan_tail(reqs, 32), reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_changing_portions(gpu, name, dtype):
    reqs = requests_for(name)
    check_plan(name, dtype, util.plan_chunks(reqs), reqs)
    check_plan(name, dtype, util.plan_chunks(reqs, sizes=(2, 2, 3, 2, 29)), reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_with_page_reuse(gpu, name, dtype):
    reqs = requests_for(name)
    for seed in (0, 1):
        plan = util.plan_mixed(reqs, seed=seed)
        assert max(len(s["entries"]) for s in plan) >= 3          # really mixed
        assert any(len(e["tokens"]) == 1 for s in plan if len(s["entries"]) > 1 for e in s["entries"])
        peak = util.live_tokens_peak(plan)
        eng, _ = check_plan(name, dtype, plan, reqs, max_tokens=peak, max_requests=4)
        pool = eng.manager.groups[0].pool
        assert pool.allocations > pool.num_pages, "the pool was so large that no page was used again"


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("C", "float32"), ("B", "bfloat16")])
def test_splits_agree_with_each_other(gpu, name, dtype):
    """The same logits whatever the cutting: bitwise in float32 where the kernels keep one order
    of summation per position, to rounding in bfloat16."""
    reqs = requests_for(name)
    eng = make_engine(name, dtype)
    whole = util.run_plan(eng, util.plan_whole(reqs))
    for plan in (util.plan_tail(reqs), util.plan_chunks(reqs), util.plan_mixed(reqs, seed=3)):
        other = util.run_plan(eng, plan)
        for rid in reqs:
            if dtype == "float32":
                assert torch.equal(whole[rid], other[rid]), f"{rid}: float32 logits depend on the cutting"
            else:
                util.assert_close_bf16(other[rid], whole[rid], rid, rms=0.02)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decode(gpu, dtype):
    """300 tokens one by one after a short prompt: crosses key tiles and many pages."""
    name = "A"
    toks = util.rand_tokens(330, util.TINY_A["vocab_size"], 77)
    reqs = {"long": toks}
    check_plan(name, dtype, util.plan_tail(reqs, 300), reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(gpu, name, dtype):
    """Positions 0, 1, 2 fed one by one, and prompts of one and two tokens."""
    V = util.CONFIGS[name][0]["vocab_size"]
    reqs = {"one": util.rand_tokens(1, V, 1), "two": util.rand_tokens(2, V, 2), "three": util.rand_tokens(3, V, 3)}
    check_plan(name, dtype, util.plan_whole(reqs), reqs)
    check_plan(name, dtype, util.plan_tail(reqs, 3), reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(gpu, dtype, tmp_path):
    """bin/trace_run as a child process gives what the engine gives in this process."""
    name = "B"
    reqs = requests_for(name)
    plan = util.plan_mixed(reqs, seed=5)
    peak = util.live_tokens_peak(plan)
    folder = util.model_folder(name, stored_for(dtype))
    got = util.run_trace_run(folder, dtype, plan, peak, str(tmp_path / "out"))
    eng = make_engine(name, dtype, max_tokens=peak)
    here = util.run_plan(eng, plan)
    for rid, toks in reqs.items():
        util.assert_close(dtype, got[rid], util.expected(name, toks, stored_for(dtype)), rid)
        assert torch.equal(got[rid], here[rid])


def test_out_of_pages_leaves_everything_as_it_was(gpu):
    from tuff_amd.cache.manager import OutOfPages
    from tuff_amd.engine.batch import StepEntry
    eng = make_engine("A", "float32", max_tokens=64)
    eng.begin("a")
    eng.begin("b")
    eng.step([StepEntry("a", list(range(40)), [39])])
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1], [0]), StepEntry("b", list(range(30)), [29])])
    assert eng.length("a") == 40 and eng.length("b") == 0
    eng.manager.check()
    eng.step([StepEntry("a", [1], [0]), StepEntry("b", list(range(10)), [9])])
    eng.manager.check()


def test_a_step_that_fails_midway_breaks_its_requests_and_no_others(gpu, monkeypatch):
    """A part raises after the first layers ran (as a refused launch does): the step's requests are refused from
    then on, whatever they hold being inconsistent (a conv state that moved on), until they are ended; the pages'
    book-keeping stays sound; a request that was not in the step goes on to the right logits; through the entry
    point, the failed requests end with the reason and the others finish."""
    from tuff_amd.engine.batch import StepEntry
    from tuff_amd.engine.engine import StepFailed
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.TINY_A["vocab_size"]
    toks = {k: util.rand_tokens(30, V, 40 + i) for i, k in enumerate("abc")}
    eng = make_engine("A", "float32", max_tokens=256, use_graphs=False)
    for k in "abc":
        eng.begin(k)
    eng.step([StepEntry("a", toks["a"][:10], []), StepEntry("c", toks["c"][:10], [])])
    last = eng.model.blocks[-1]
    real = last.forward
    calls = {"n": 0}

    def failing(*a, **kw):
        calls["n"] += 1
        if calls["n"] == 1:
            raise RuntimeError("launch refused")
        return real(*a, **kw)
    monkeypatch.setattr(last, "forward", failing)
    with pytest.raises(StepFailed) as e:
        eng.step([StepEntry("a", toks["a"][10:20], [9]), StepEntry("b", toks["b"][:7], [6])])
    assert sorted(e.value.requests) == ["a", "b"] and isinstance(e.value.__cause__, RuntimeError)
    eng.manager.check()
    assert eng.length("a") == 10 and eng.length("b") == 0
    with pytest.raises(ValueError, match="failed midway"):
        eng.step([StepEntry("a", toks["a"][10:20], [9])])
    got = eng.step([StepEntry("c", toks["c"][10:], list(range(20)))])           # untouched by the failure
    util.assert_close_f32(got.cpu(), util.plain_logits("A", toks["c"], "float32")[10:], "c")
    eng.end("a")
    eng.begin("a")                                                             # ended and begun again: as new
    got = eng.step([StepEntry("a", toks["a"], list(range(30)))])
    util.assert_close_f32(got.cpu(), util.plain_logits("A", toks["a"], "float32"), "a again")
    for k in "abc":
        eng.end(k)
    # the entry point
    llm = LLM(engine=eng, max_num_seqs=4, max_batched_tokens=12)
    calls["n"] = -4                                                            # the sixth step fails
    sched = llm.new_scheduler()
    from tuff_amd.engine.scheduler import Request
    reqs = [Request(k, toks[k][:9], SamplingParams(max_new_tokens=8)) for k in "abc"]
    for r in reqs:
        sched.add(r)
    with pytest.raises(StepFailed):
        llm.run(sched)
    failed = [r for r in reqs if (r.finish_reason or "").startswith("error: launch refused")]
    assert failed and all(r.status == "finished" and -1 not in r.output for r in failed)
    llm.run(sched)                                                             # whoever was not in that step goes on
    assert all(r.status == "finished" for r in reqs) and not eng.manager.live()
    eng.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_decode_steps_equal_eager_steps(gpu, dtype):
    """Steps of single tokens are recorded into a graph and replayed.  Every replay, with eager
    steps of other shapes and synchronisations in between, gives exactly what an engine without
    graphs gives; a context that outgrows the recorded table width gets a new recording."""
    name = "A"
    V = util.TINY_A["vocab_size"]
    reqs = {"x": util.rand_tokens(1050, V, 1), "y": util.rand_tokens(120, V, 2), "z": util.rand_tokens(40, V, 3)}
    steps = []
    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})
    fed = {k: 0 for k in reqs}
    def portion(rid, n):
        t = reqs[rid][fed[rid]:fed[rid] + n]
        fed[rid] += n
        return {"id": rid, "tokens": t, "want": [len(t) - 1]}
    add([portion("x", 1000), portion("y", 50)])
    for i in range(45):
        if i == 10:
            add([portion("z", 20)])                                  # an eager step of another shape in between
        if i == 20:
            add([portion("x", 1), portion("y", 1), portion("z", 5)])  # mixed: not recorded
        add([portion("x", 1), portion("y", 1)] + ([portion("z", 1)] if 12 <= i < 20 else []))
    add([portion("x", 1)], end=["x", "y", "z"])
    assert fed["x"] > 1024                                            # x crossed the 64-block table width
    eager = make_engine(name, dtype, max_tokens=2048, use_graphs=False)
    want = util.run_plan(eager, steps)
    eng = make_engine(name, dtype, max_tokens=2048)
    assert eng.use_graphs
    got = util.run_plan(eng, steps)
    assert eng.graph_replays >= 30 and len(eng._graphs) >= 3
    assert eager.graph_replays == 0
    for rid in reqs:
        a, b = got[rid], want[rid]
        mask = ~torch.isnan(b[:, 0])
        assert torch.equal(torch.isnan(a[:, 0]), torch.isnan(b[:, 0]))
        assert torch.equal(a[mask], b[mask]), rid
    full = util.expected(name, reqs["y"][:fed["y"]], stored_for(dtype))
    mask = ~torch.isnan(got["y"][:, 0])
    util.assert_close(dtype, got["y"][mask], full[mask], "y")


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("A", "bfloat16"), ("B", "bfloat16")])
def test_steps_with_portions_recorded_in_sections_equal_eager_steps(gpu, name, dtype, monkeypatch):
    """A number of tokens that keeps coming is recorded as graphs with the attention and the head run
    eagerly in between.  Steps of that size with other requests, other portions, other wanted rows and
    other places in the cache, with steps of other sizes and of single tokens in between, give exactly
    what an engine that records nothing gives; so do the tokens decoded afterwards out of the cache
    and the conv states those steps left."""
    from tuff_amd.engine.engine import Engine
    V = util.CONFIGS[name][0]["vocab_size"]
    reqs = {k: util.rand_tokens(n, V, 10 + i) for i, (k, n) in enumerate(
        [("a", 300), ("b", 220), ("c", 130), ("d", 90), ("e", 75)])}
    steps, fed = [], {k: 0 for k in reqs}
    def portion(rid, n, want=True):
        t = reqs[rid][fed[rid]:fed[rid] + n]
        fed[rid] += n
        return {"id": rid, "tokens": t, "want": ([len(t) - 1] if want else [])}
    def add(entries, end=()):
        assert all(e["tokens"] for e in entries)
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})
    T = 70
    add([portion("a", T)])                                                # T tokens: first
    add([portion("a", 40), portion("b", 30, want=False)])                 # second
    add([portion("b", 69), portion("c", 1)])                              # third: recorded and replayed
    add([portion("c", 1), portion("a", 1), portion("b", 1)])              # single tokens in between
    add([portion("a", 1), portion("c", 60), portion("b", 1), portion("d", 8, want=False)])   # replay, four requests
    add([portion("d", 33)])                                               # another size
    add([portion("e", 2, want=False), portion("a", 1), portion("b", 60), portion("c", 1), portion("d", 6)])
    add([portion("e", 70)], end=["e"])                                    # e's pages and slot go back ...
    reqs["f"] = util.rand_tokens(100, V, 99); fed["f"] = 0
    add([portion("f", 66), portion("a", 1), portion("c", 3)])             # ... and are used again
    for _ in range(4):
        add([portion(k, 1) for k in "abcdf"])
    add([portion("a", 64), portion("f", 6)], end=list("abcdf"))
    counts = [sum(len(e["tokens"]) for e in s["entries"]) for s in steps]
    assert counts.count(T) == 8
    eager = make_engine(name, dtype, max_tokens=1024, use_graphs=False, max_requests=5)
    want = util.run_plan(eager, steps)
    eng = make_engine(name, dtype, max_tokens=1024, max_requests=5)
    assert eng.record_portions
    got = util.run_plan(eng, steps)
    assert eng.section_replays == 6 and eager.section_replays == 0
    eng.manager.check()
    for rid in reqs:
        a, b = got[rid], want[rid]
        assert torch.equal(torch.isnan(a[:, 0]), torch.isnan(b[:, 0]))
        mask = ~torch.isnan(b[:, 0])
        assert torch.equal(a[mask], b[mask]), rid
    full = util.expected(name, reqs["b"][:fed["b"]], stored_for(dtype))
    mask = ~torch.isnan(got["b"][:, 0])
    util.assert_close(dtype, got["b"][mask], full[mask], "b")


def test_the_threshold_for_recording_comes_down_again(gpu, monkeypatch):
    """Many sizes taking turns push recordings out before they are used again, and a size then has to come more
    often to be recorded; a steady stream of one size afterwards is recorded all the same, and the threshold comes
    down while its replays go through."""
    from tuff_amd.engine.batch import StepEntry
    from tuff_amd.engine.engine import Engine
    monkeypatch.setattr(Engine, "MAX_SECTIONED", 1)
    monkeypatch.setattr(Engine, "SECTIONS_CALM_REPLAYS", 4)
    monkeypatch.setattr(Engine, "SECTIONS_SEEN_KEPT", 3)
    V = util.TINY_A["vocab_size"]
    eng = make_engine("A", "bfloat16", max_tokens=4096)
    eng.begin("r")
    rng_tokens = util.rand_tokens(4000, V, 3)
    at = 0

    def feed(n):
        nonlocal at
        eng.step([StepEntry("r", rng_tokens[at:at + n], [n - 1])])
        at += n
    for n in (5, 6, 7, 8):                     # each size until it is recorded, then never again: every recording is
        for _ in range(eng._record_at):        # pushed out after its one replay, and the threshold doubles
            feed(n)
    raised = eng._record_at
    assert raised > Engine.SECTIONS_RECORD_AT and len(eng._sectioned_seen) <= 3
    before = eng.section_replays
    for _ in range(raised + 12):               # a steady stream of one size
        feed(9)
    assert eng.section_replays - before >= 12 and eng._record_at < raised
    eng.end("r")


@pytest.mark.parametrize("name", ["A", "E"])
def test_recorded_steps_whose_every_row_is_wanted_equal_eager_steps(gpu, name):
    """Teacher forcing in portions of at most 64 tokens with every row wanted: the last block's product leaves
    the final norm's operand and row sums for the head.  The head runs outside of what is recorded; at a replay it
    must find that operand as in an eager step (it once found nothing and took another product: other bits)."""
    V = util.CONFIGS[name][0]["vocab_size"]
    toks = util.rand_tokens(40 * 9, V, 5)
    steps = [{"step": i, "entries": [{"id": "t", "tokens": toks[40 * i:40 * i + 40], "want": list(range(40))}], "end": []}
             for i in range(9)]
    steps[-1]["end"] = ["t"]
    eager = make_engine(name, "bfloat16", max_tokens=512, use_graphs=False)
    want = util.run_plan(eager, steps)
    eng = make_engine(name, "bfloat16", max_tokens=512)
    assert eng.record_portions
    got = util.run_plan(eng, steps)
    assert eng.section_replays >= 6
    assert torch.equal(got["t"], want["t"])
    util.assert_close("bfloat16", got["t"], util.expected(name, toks, "bfloat16"), "teacher forcing")


def test_recordings_are_dropped_and_made_again(gpu, monkeypatch):
    """Room for one recording of each kind: sizes that take turns push each other out and are recorded
    again, and every step still equals the eager one."""
    from tuff_amd.engine.engine import Engine
    monkeypatch.setattr(Engine, "MAX_SECTIONED", 1)
    monkeypatch.setattr(Engine, "MAX_GRAPHS", 1)
    V = util.TINY_A["vocab_size"]
    reqs = {k: util.rand_tokens(800, V, 30 + i) for i, k in enumerate("abc")}
    steps, fed = [], {k: 0 for k in reqs}
    def portion(rid, n):
        t = reqs[rid][fed[rid]:fed[rid] + n]
        fed[rid] += n
        assert len(t) == n
        return {"id": rid, "tokens": t, "want": [len(t) - 1]}
    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})
    for rnd in range(3):
        for _ in range(4):
            add([portion("a", 40), portion("b", 10)])          # 50 tokens
        for _ in range(2):
            add([portion("a", 1), portion("b", 1)])            # two single tokens
        for _ in range(4):
            add([portion("b", 1), portion("c", 59)])           # 60 tokens
        for _ in range(2):
            add([portion(k, 1) for k in "abc"])                # three single tokens
    add([portion("a", 1)], end=list("abc"))
    eager = make_engine("A", "bfloat16", max_tokens=2560, use_graphs=False)
    want = util.run_plan(eager, steps)
    eng = make_engine("A", "bfloat16", max_tokens=2560)
    got = util.run_plan(eng, steps)
    # a size is recorded when it has come three times: in the first round its third and fourth step replay, later all four
    assert eng.section_replays == 2 * 2 + 2 * 2 * 4 and len(eng._sectioned) == 1 and len(eng._graphs) == 1
    assert eng.graph_replays == 3 * 2 * 1
    for rid in reqs:
        mask = ~torch.isnan(want[rid][:, 0])
        assert torch.equal(got[rid][mask], want[rid][mask]), rid


def test_sizes_that_push_each_other_out_are_recorded_less_and_less_often(gpu, monkeypatch):
    """Three sizes take turns, one step each, with room for one recording: a recording is pushed out before
    it is used again, so the engine asks for more and more returns of a size before it records it; the
    steps still equal the eager ones."""
    from tuff_amd.engine.engine import Engine
    monkeypatch.setattr(Engine, "MAX_SECTIONED", 1)
    V = util.TINY_A["vocab_size"]
    reqs = {k: util.rand_tokens(2200, V, 40 + i) for i, k in enumerate("ab")}
    steps, fed = [], {k: 0 for k in reqs}
    def portion(rid, n):
        t = reqs[rid][fed[rid]:fed[rid] + n]
        fed[rid] += n
        assert len(t) == n
        return {"id": rid, "tokens": t, "want": [n - 1]}
    for rnd in range(14):
        for n in (40, 50, 60):
            steps.append({"step": len(steps), "entries": [portion("a", n - 10), portion("b", 10)], "end": []})
    steps[-1]["end"] = ["a", "b"]
    eager = make_engine("A", "bfloat16", max_tokens=4480, use_graphs=False)
    want = util.run_plan(eager, steps)
    eng = make_engine("A", "bfloat16", max_tokens=4480)
    got = util.run_plan(eng, steps)
    # recorded at every step from the third round on it would be 36 times
    assert 3 <= eng.section_recordings <= 8 and eng.section_replays > eng.section_recordings
    for rid in reqs:
        mask = ~torch.isnan(want[rid][:, 0])
        assert torch.equal(got[rid][mask], want[rid][mask]), rid


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_token_ids_taken_from_the_device(gpu, dtype):
    """A step may take some of its token ids from a vector on the device (the sampler's output of
    the step before) instead of from its entries: a step of portions beside single tokens, and a
    recorded step of single tokens, give exactly what they give with the ids in the entries."""
    from tuff_amd.engine.batch import StepEntry
    V = util.TINY_B["vocab_size"]
    toks = {k: util.rand_tokens(40, V, 5 + i) for i, k in enumerate("abc")}
    drawn = torch.tensor([toks["c"][20], 0, toks["a"][20], toks["b"][21], toks["a"][21]], dtype=torch.int32, device=gpu)

    def steps(eng, from_device):
        for k in toks:
            eng.begin(k)
        eng.step([StepEntry(k, toks[k][:20], []) for k in "ab"])
        hide = (lambda t: 0) if from_device else (lambda t: t)
        # c's portion between two single tokens, then single tokens in another order than `drawn`
        first = [StepEntry("a", [hide(toks["a"][20])], [0]), StepEntry("c", toks["c"][:20], [19]),
                 StepEntry("b", toks["b"][20:21], [0])]
        second = [StepEntry("b", [hide(toks["b"][21])], [0]), StepEntry("c", [hide(toks["c"][20])], [0]),
                  StepEntry("a", [hide(toks["a"][21])], [0])]
        out = [eng.step(first, (drawn, [0], [2]) if from_device else None).float().cpu(),
               eng.step(second, (drawn, [0, 1, 2], [3, 0, 4]) if from_device else None).float().cpu()]
        for k in toks:
            eng.end(k)
        return out

    for graphs in (False, True):
        eng = make_engine("B", dtype, use_graphs=graphs)
        want, got = steps(eng, False), steps(eng, True)
        assert all(torch.equal(w, g) for w, g in zip(want, got))
        assert not graphs or eng.graph_replays >= 1
    util.assert_close(dtype, got[1][2:], util.expected("B", toks["a"][:22], stored_for(dtype))[21:], "a")
    with pytest.raises(ValueError, match="out of range"):
        eng.begin("a")
        eng.step([StepEntry("a", [1, 2], [])], (drawn, [2], [0]))
    assert eng.length("a") == 0
    eng.end("a")


def test_layers_of_full_size_float32_against_the_plain_implementation(gpu):
    """Layers with the sizes of a 1.2B model, float32, against the plain implementation: whole, a
    head then single tokens, and two requests mixed in portions."""
    name = "F"
    V = util.FULL_SIZE_LAYERS["vocab_size"]
    reqs = {"a": util.rand_tokens(70, V, 21), "b": util.rand_tokens(37, V, 22)}
    from tuff_amd.engine.engine import Engine
    folder = util.model_folder(name, "bfloat16")            # both paths read these bfloat16 weights
    eng = Engine.from_folder(folder, dtype="float32", page_size=16, max_tokens=256)
    want = {rid: util.expected(name, toks, "bfloat16") for rid, toks in reqs.items()}
    first = None
    for plan in (util.plan_whole(reqs), util.plan_tail(reqs, 8), util.plan_mixed(reqs, seed=2, decode_tail=6),
                 util.plan_chunks(reqs)):
        got = util.run_plan(eng, plan)
        eng.manager.check()
        for rid in reqs:
            util.assert_close_f32(got[rid], want[rid], f"full-size float32 {rid}")
        first = first or got
        for rid in reqs:                                    # and bitwise the same however the requests were cut
            assert torch.equal(got[rid], first[rid]), f"full-size float32 {rid}: logits depend on the cutting"
    del eng
    eng16 = Engine.from_folder(folder, dtype="bfloat16", page_size=16, max_tokens=256)
    got16 = util.run_plan(eng16, util.plan_whole(reqs))
    for rid in reqs:
        util.assert_close_bf16(got16[rid], want[rid], f"full-size bfloat16 {rid}")


def test_layers_of_full_size_bfloat16_against_float32(gpu):
    """Layers with the sizes of a 1.2B model (hidden 2048, 32 query and 8 kv heads of 64, feed-forward
    8192, vocabulary 65536; two conv layers and an attention layer): the bfloat16 kernels chosen at
    these sizes (large matrix tiles, portions of several query blocks, single tokens over several
    key partitions) against the float32 path, which the tiny configurations pin to the plain
    implementation.  Both engines hold the same weights (made in bfloat16)."""
    from tuff_amd.engine.batch import StepEntry
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models.registry import config_from_dict
    cfg = config_from_dict(dict(
        architectures=["Lfm2ForCausalLM"], num_hidden_layers=3, layer_types=["conv", "conv", "full_attention"],
        hidden_size=2048, num_attention_heads=32, num_key_value_heads=8, block_ff_dim=12288,
        block_auto_adjust_ff_dim=True, block_multiple_of=256, block_ffn_dim_multiplier=1.0, vocab_size=65536,
        rope_theta=1000000.0, conv_L_cache=3, norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=8192))
    assert cfg.ffn_dim == 8192
    tokens = util.rand_tokens(700, cfg.vocab_size, 5)
    other = util.rand_tokens(90, cfg.vocab_size, 6)
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_config(cfg, 3, dtype=dtype, page_size=16, num_pages=64, max_requests=2)
        got = []
        eng.begin("a")
        eng.begin("b")
        got.append(eng.step([StepEntry("a", tokens[:600], [0, 299, 599])]))          # one large portion
        got.append(eng.step([StepEntry("a", tokens[600:690], [89]), StepEntry("b", other[:80], [79])]))
        for i in range(690, 700):                                                     # single tokens, two requests
            got.append(eng.step([StepEntry("a", [tokens[i]], [0]), StepEntry("b", [other[i - 610]], [0])]))
        outs[dtype] = torch.cat([g.float().cpu() for g in got])
        eng.end("a")
        eng.end("b")
        del eng
        torch.cuda.empty_cache()
    util.assert_close_bf16(outs["bfloat16"], outs["float32"], "full-size layers")
    # and the first choice agrees wherever float32 is not close to a tie
    top = torch.topk(outs["float32"], 2, dim=-1).values
    clear = (top[:, 0] - top[:, 1]) > 0.05 * float(outs["float32"].std())
    assert (outs["bfloat16"].argmax(-1) == outs["float32"].argmax(-1))[clear].all()


def test_decode_of_64_requests_at_8192_keys_against_float32(gpu):
    """The benchmark's largest launches, whole: 64 requests with 8,191 tokens each in the cache bring one token.
    The attention then runs 16,384 workgroups a layer (a wave a partition of 256 keys, the kv head changing fastest
    in their order, keys through LDS) and the products take 64 rows.  Against the float32 path on the same cache:
    the bfloat16 engine computes the prompts, its keys, values and conv states are copied (exactly) into a float32
    engine, and both run the step.  With random weights 8,192 keys weigh about the same, and the attention adds a
    thirtieth of what the feed-forwards put into the residual stream: a partition more or less would change nothing
    one could see.  So one value in every partition of every request is made fifty times as large as the others
    (each is then a third of its request's attention output), and the attention's output projection thirty-two times
    as large (the attention then adds about what the stream holds)."""
    import ctypes
    import random
    from tuff_amd.cache.storage import PagedKVView
    from tuff_amd.csrc import ops
    from tuff_amd.engine.batch import StepEntry
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models.registry import build_model, config_from_dict
    from tuff_amd.weights.random_init import random_weights
    cfg = config_from_dict(util.FULL_SIZE_LAYERS)
    R, ctx, ps = 64, 8192, 16
    rng = random.Random(5)
    kw = dict(page_size=ps, num_pages=R * ctx // ps + 8, max_requests=R)
    engines = []
    for dtype in (torch.bfloat16, torch.float32):
        model = build_model(cfg)
        weights = random_weights(model.weight_decls(), 7, dtype, gpu)
        weights["model.layers.1.self_attn.out_proj.weight"] *= 32.0          # (a power of two: exact in either type)
        engines.append(Engine(model, weights, dtype=dtype, **kw))
    a, b = engines
    lib = ops.load("attention_mfma")
    lib.tuff_attention_stage_k_waves.argtypes, lib.tuff_attention_stage_k_waves.restype = [ctypes.c_int], ctypes.c_int
    assert R * (ctx // ops.ATTN_PARTITION) * cfg.num_key_value_heads >= lib.tuff_attention_stage_k_waves(-1)
    last = []
    for r in range(R):
        toks = util.rand_tokens(ctx, cfg.vocab_size, 900 + r)
        a.begin(r)
        b.begin(r)
        for i in range(0, ctx - 1, 2048):
            a.step([StepEntry(r, toks[i:min(i + 2048, ctx - 1)], [])])
        b.manager.extend(r, ctx - 1)
        assert a.manager.block_table(r, 0) == b.manager.block_table(r, 0)
        last.append(toks[-1])
    loud = []                                          # (page, offset) of one position in every partition of every request
    for r in range(R):
        table = a.manager.block_table(r, 0)
        for part in range(ctx // ops.ATTN_PARTITION):
            pos = min(part * ops.ATTN_PARTITION + rng.randrange(ops.ATTN_PARTITION), ctx - 2)
            loud.append((table[pos // ps], pos % ps))
    pages = torch.tensor([p for p, _ in loud], device=gpu)
    offs = torch.tensor([o for _, o in loud], device=gpu)
    for e, va in a.storage.views.items():
        vb = b.storage.views[e]
        if isinstance(va, PagedKVView):
            va.v[pages, :, :, offs] *= 50.0
            vb.k.copy_(va.k)
            vb.v.copy_(va.v)
        else:
            vb.state.copy_(va.state)
    entries = [StepEntry(r, [last[r]], [0]) for r in range(R)]
    got = a.step(entries).float().cpu()
    states_before = {e: vb.state.clone() for e, vb in b.storage.views.items() if not isinstance(vb, PagedKVView)}
    want = b.step(entries).float().cpu()
    assert torch.isfinite(want).all()
    util.assert_close_bf16(got, want, "64 requests at 8,192 keys", rms=0.02)
    # what a loud value is worth: without one of them (request 3, its partition 17) the float32 logits of that request
    # move by far more than the tolerance, so a partition lost or taken twice would show
    b.manager.truncate(3, ctx - 1)
    page, off = loud[3 * (ctx // ops.ATTN_PARTITION) + 17]
    for e, vb in b.storage.views.items():
        if isinstance(vb, PagedKVView):
            vb.v[page, :, :, off] /= 50.0
        else:
            vb.state.copy_(states_before[e])               # the conv states as they were before the step
    again = b.step([entries[3]]).float().cpu()
    other = again
    spread = float(want[3].double().pow(2).mean().sqrt())
    assert float((other[0].double() - want[3].double()).pow(2).mean().sqrt()) > 0.05 * spread


def test_the_benchmarked_model(gpu):
    """The model bench.py times (16 layers of the 1.2B shape, random weights of its seed), three requests of 200, 64
    and 141 tokens: the float32 engine against the plain implementation in float64, the same bits whole, with the
    last 32 tokens one by one, and mixed in portions beside single tokens; the bfloat16 engine under the same three
    plans against the plain implementation, its error measured with the plain implementation's rounding model; the
    first choice agrees wherever float32 is not close to a tie."""
    import bench
    from plain.lfm2_plain import forward_logits
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models.registry import build_model
    from tuff_amd.weights.random_init import random_weights
    cfg = bench.shape_config(bench.SHAPE["num_hidden_layers"])
    assert cfg.num_hidden_layers == 16 and build_model(cfg).num_parameters() == 1170340608
    V = cfg.vocab_size
    reqs = {"a": util.rand_tokens(200, V, 61), "b": util.rand_tokens(64, V, 62), "c": util.rand_tokens(141, V, 63)}
    plans = {"whole": util.plan_whole(reqs), "tail": util.plan_tail(reqs, 32),
             "mixed": util.plan_mixed(reqs, seed=8, decode_tail=10)}
    model = build_model(cfg)
    weights = random_weights(model.weight_decls(), bench.SEED, torch.float32, gpu)
    eng = Engine(model, weights, dtype="float32", page_size=16, max_tokens=1024, max_requests=4, poison_cache=True)
    got32 = {k: util.run_plan(eng, p) for k, p in plans.items()}
    for k in ("tail", "mixed"):
        for rid in reqs:
            assert torch.equal(got32[k][rid], got32["whole"][rid]), f"float32, {k}, {rid}: logits depend on the cutting"

    class AsFloat64(dict):                      # one tensor at a time: the whole model in float64 would be 9 GB
        def __getitem__(self, name):
            return dict.__getitem__(self, name).double()

        def __contains__(self, name):
            return dict.__contains__(self, name)
    raw = dict(cfg.to_dict(), layer_types=["conv" if cfg.is_conv(i) else "full_attention" for i in range(16)])
    host = AsFloat64({k: v.cpu() for k, v in weights.items()})
    want = {rid: util.expected_of(raw, host, toks) for rid, toks in reqs.items()}
    for rid in reqs:
        util.assert_close_f32_deep(got32["whole"][rid], want[rid].want, f"benchmarked model, float32 against plain, {rid}")
    del eng, weights, model, host
    torch.cuda.empty_cache()

    eng16 = Engine.from_config(cfg, bench.SEED, dtype="bfloat16", page_size=16, max_tokens=1024, max_requests=4,
                               poison_cache=True)
    for k, plan in plans.items():
        got16 = util.run_plan(eng16, plan)
        for rid in reqs:
            ref = got32["whole"][rid]
            util.assert_close_bf16(got16[rid], want[rid], f"benchmarked model, bfloat16 {k} {rid}")
            # the first choice agrees wherever float32's two best are further apart than the row's own rounding noise
            # can bridge (six times the RMS difference of the row: the two logits' errors are independent)
            top = torch.topk(ref, 2, dim=-1).values
            noise = (got16[rid].double() - ref.double()).pow(2).mean(-1).sqrt()
            clear = (top[:, 0] - top[:, 1]).double() > 6 * noise
            assert clear.sum() >= len(clear) // 4                      # random weights: many rows are near-ties
            assert (got16[rid].argmax(-1) == ref.argmax(-1))[clear].all(), (k, rid)


def random_configuration(seed: int) -> dict:
    """A small configuration whose every size and option is drawn from the seed."""
    import random
    rng = random.Random(seed)
    heads = rng.choice([1, 2, 3, 4, 6, 8])
    kv = rng.choice([h for h in range(1, heads + 1) if heads % h == 0])
    hd = rng.choice([4, 12, 16, 20, 24, 32, 40, 48, 64, 80, 100, 128])
    layers = rng.randint(2, 5)
    types = [rng.choice(["conv", "full_attention"]) for _ in range(layers)]
    types[rng.randrange(layers)] = "full_attention"
    types[(types.index("full_attention") + 1) % layers] = "conv"
    return dict(
        architectures=["Lfm2ForCausalLM"], num_hidden_layers=layers, layer_types=types,
        hidden_size=heads * hd, num_attention_heads=heads, num_key_value_heads=kv,
        block_ff_dim=rng.choice([40, 72, 100, 136, 200, 333]), block_auto_adjust_ff_dim=False,
        vocab_size=rng.randint(90, 1500), rope_theta=rng.choice([1e4, 5e5, 1e6]), conv_L_cache=rng.randint(2, 5),
        norm_eps=rng.choice([1e-5, 1e-6, 3e-6]), tie_word_embeddings=rng.random() < 0.5, max_position_embeddings=512)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15])
def test_configurations_drawn_at_random(gpu, tmp_path, seed, dtype):
    """Configurations whose sizes nobody chose (head counts and sizes, groups, widths that are no
    multiple of 8, vocabulary, conv length, layer order), under the mixed plan, against the plain
    implementation."""
    import random
    from plain.lfm2_plain import forward_logits, read_model
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models.registry import config_from_dict
    from tuff_amd.weights.random_init import write_random_model
    raw = random_configuration(seed)
    stored = stored_for(dtype)
    folder = str(tmp_path / "model")
    write_random_model(config_from_dict(raw), folder, seed, getattr(torch, stored))
    cfg, w = read_model(folder)
    rng = random.Random(seed)
    reqs = {f"q{i}": util.rand_tokens(rng.randint(3, 120), raw["vocab_size"], seed * 10 + i) for i in range(5)}
    plan = util.plan_mixed(reqs, seed=seed)
    make = lambda: Engine.from_folder(folder, dtype=dtype, page_size=rng.choice([16, 32]),
                                      max_tokens=util.live_tokens_peak(plan) + 64)
    if dtype == "bfloat16" and raw["hidden_size"] % 8:
        # the bfloat16 matrix kernels read 16 bytes at a time along the hidden size: refused, in words
        with pytest.raises(ValueError, match="multiple of 8"):
            make()
        return
    eng = make()
    got = util.run_plan(eng, plan)
    eng.manager.check()
    for rid, toks in reqs.items():
        util.assert_close(dtype, got[rid], util.expected_of(cfg, w, toks), f"seed {seed} {raw} {rid}")
