"""Generation through the entry points: greedy and seeded temperature sampling of several
requests at once against the plain implementation, preemption, the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import util
from plain import lfm2_plain as plain
from plain.sampler_plain import PlainSampler

pytestmark = pytest.mark.gpu


def plain_generate(name, prompt, n, stored, sampler=None):
    """Token by token with the plain model; returns ids and, for greedy, the top-1/top-2 margins."""
    cfg, w = util.plain_model(name, stored)
    ids, out, margins = list(prompt), [], []
    for _ in range(n):
        row = plain.forward_logits(cfg, w, ids)[-1]
        if sampler is None:
            top = torch.topk(row, 2).values
            margins.append(float(top[0] - top[1]))
            t = int(torch.nonzero(row == row.max())[0])
        else:
            t = sampler.sample(row.float().numpy())
            margins.append(None)
        out.append(t)
        ids.append(t)
    return out, margins


def agree_up_to_near_ties(got, want, margins, tie):
    """Equal until the first step at which the plain model's top two logits are closer than `tie`
    (cf. tools/lfm25_gate.py:54-73: the greedy prefix is cut at the first near-tie)."""
    for i, (g, w) in enumerate(zip(got, want)):
        if g != w:
            assert margins[i] < tie, f"step {i}: got {g}, plain {w}, margin {margins[i]:.2e}"
            return i
    return len(want)


@pytest.mark.parametrize("dtype,stored,tie", [("float32", "float32", 2e-5), ("bfloat16", "bfloat16", 2e-2)])
def test_greedy_generation_tiny_a(gpu, dtype, stored, tie):
    """Tiny A: prompts of 7, 13 and 21 tokens, 16 greedy tokens each, all at once."""
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.TINY_A["vocab_size"]
    prompts = [util.rand_tokens(n, V, 10 + n) for n in (7, 13, 21)]
    llm = LLM(util.model_folder("A", stored), dtype=dtype, max_num_seqs=4, max_batched_tokens=16, ctx_size=128)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=16))
    total = 0
    for p, o in zip(prompts, outs):
        want, margins = plain_generate("A", p, 16, stored)
        assert len(o.token_ids) == 16 and o.finish_reason == "length"
        total += agree_up_to_near_ties(o.token_ids, want, margins, tie)
    assert total >= 24                       # most of the 48 tokens are compared, not cut away by ties
    assert not llm.engine.manager.live()


def test_seeded_temperature_sampling_tiny_b(gpu):
    """Tiny B: prompts of 1, 5, 33, 64 and 100 tokens; temperature 0.8 with per-request seeds next to
    greedy requests, in float32, equal to the plain model with the plain sampler."""
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.TINY_B["vocab_size"]
    prompts = [util.rand_tokens(n, V, 20 + n) for n in (1, 5, 33, 64, 100)]
    params = [SamplingParams(temp=0.8, seed=100 + i, max_new_tokens=12) if i % 2 == 0 else SamplingParams(max_new_tokens=12)
              for i in range(5)]
    llm = LLM(util.model_folder("B", "float32"), dtype="float32", max_num_seqs=4, max_batched_tokens=48, ctx_size=160)
    outs = llm.generate(prompts, params)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        sampler = PlainSampler(temp=0.8, seed=100 + i) if i % 2 == 0 else None
        want, margins = plain_generate("B", p, 12, "float32", sampler)
        if sampler is None:
            agree_up_to_near_ties(o.token_ids, want, margins, 2e-5)
        else:
            assert o.token_ids == want, i
    # the same seeds again, one request at a time: the stream does not depend on the batch
    for i in (0, 2):
        alone = llm.generate([prompts[i]], params[i])[0]
        assert alone.token_ids == outs[i].token_ids


def test_sampling_options_through_the_entry_point(gpu):
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.TINY_A["vocab_size"]
    prompt = util.rand_tokens(9, V, 3)
    llm = LLM(util.model_folder("A", "float32"), dtype="float32", ctx_size=64)
    greedy = llm.generate([prompt], SamplingParams(max_new_tokens=8))[0].token_ids
    top1 = llm.generate([prompt], SamplingParams(temp=3.0, top_k=1, seed=5, max_new_tokens=8))[0].token_ids
    assert top1 == greedy                                                     # top-k 1 is greedy whatever the draw
    cold = llm.generate([prompt], SamplingParams(temp=1e-4, seed=5, max_new_tokens=8))[0].token_ids
    assert cold == greedy                                                     # temperature -> 0+ is greedy
    p = SamplingParams(temp=1.5, top_k=50, top_p=0.9, min_p=0.01, repeat_penalty=1.3, seed=9, max_new_tokens=10)
    a = llm.generate([prompt], p)[0].token_ids
    b = llm.generate([prompt], p)[0].token_ids
    assert a == b and a != greedy
    want, _ = plain_generate("A", prompt, 10, "float32",
                             PlainSampler(temp=1.5, top_k=50, top_p=0.9, min_p=0.01, repeat_penalty=1.3, seed=9))
    assert a == want


def test_preemption_does_not_change_the_output(gpu):
    """So few pages that running requests are preempted and computed again: same tokens."""
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.TINY_A["vocab_size"]
    prompts = [util.rand_tokens(n, V, 40 + n) for n in (30, 28, 26)]
    params = [SamplingParams(temp=0.9, seed=7, max_new_tokens=40), SamplingParams(max_new_tokens=40),
              SamplingParams(temp=0.5, seed=8, max_new_tokens=40)]
    roomy = LLM(util.model_folder("A", "float32"), dtype="float32", max_num_seqs=4, ctx_size=128)
    want = [o.token_ids for o in roomy.generate(prompts, params)]
    assert roomy.last_stats["preemptions"] == 0
    tight = LLM(util.model_folder("A", "float32"), dtype="float32", max_num_seqs=4, ctx_size=128, num_pages=9)
    outs = tight.generate(prompts, params)
    assert tight.last_stats["preemptions"] >= 1
    assert [o.token_ids for o in outs] == want
    assert sum(o.preemptions for o in outs) == tight.last_stats["preemptions"]
    tight.engine.manager.check()
    assert not tight.engine.manager.live()


def test_bfloat16_tokens_change_with_the_neighbours_only_at_near_ties(gpu, capsys):
    """In bfloat16 the kernels a token goes through depend on the step it is in (products of up to 16,
    up to 64 or more rows, single-token or portion attention), so its logits carry another rounding
    with other neighbours.  Greedy tokens of six requests run together under a small budget, again
    with so few pages that requests are preempted and computed again, and each alone: where a
    request's tokens differ from its tokens alone, the plain model's top two logits at that step
    (along the tokens it produced alone) are within the bound the logits' rounding allows."""
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    name, n_new, tie = "B", 40, 2e-2
    V = util.CONFIGS[name][0]["vocab_size"]
    prompts = [util.rand_tokens(n, V, 300 + n) for n in (5, 37, 18, 70, 9, 52)]
    p = SamplingParams(max_new_tokens=n_new)
    folder = util.model_folder(name, "bfloat16")
    alone_llm = LLM(folder, dtype="bfloat16", max_num_seqs=1, ctx_size=128)
    alone = [alone_llm.generate([q], p)[0].token_ids for q in prompts]
    cfg, w = util.plain_model(name, "bfloat16")
    margins = []
    for q, toks in zip(prompts, alone):
        rows = plain.forward_logits(cfg, w, q + toks)[len(q) - 1:-1]
        top = torch.topk(rows, 2, dim=-1).values
        margins.append((top[:, 0] - top[:, 1]).tolist())
    together = LLM(folder, dtype="bfloat16", max_num_seqs=6, max_batched_tokens=24, ctx_size=128)
    tight = LLM(folder, dtype="bfloat16", max_num_seqs=6, max_batched_tokens=24, ctx_size=128, num_pages=20)
    report = {}
    for tag, llm in (("together", together), ("tight pool", tight)):
        outs = [o.token_ids for o in llm.generate(prompts, p)]
        diverged = 0
        for i, (got, want) in enumerate(zip(outs, alone)):
            assert len(got) == n_new
            cut = agree_up_to_near_ties(got, want, margins[i], tie)
            diverged += cut < n_new
        report[tag] = diverged
        llm.engine.manager.check()
        assert not llm.engine.manager.live()
    assert tight.last_stats["preemptions"] >= 1
    with capsys.disabled():
        print(f"\n[bf16 neighbours] requests whose greedy tokens left their tokens alone at a near-tie, of {len(prompts)}: {report}")


def test_eos_stops_a_request(gpu):
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.TINY_A["vocab_size"]
    prompt = util.rand_tokens(11, V, 9)
    llm = LLM(util.model_folder("A", "float32"), dtype="float32", ctx_size=64)
    free = llm.generate([prompt], SamplingParams(max_new_tokens=10))[0].token_ids
    llm.engine.model.eos_token_id = free[3]
    out = llm.generate([prompt], SamplingParams(max_new_tokens=10))[0]
    cut = free.index(free[3]) + 1
    assert out.token_ids == free[:cut] and out.finish_reason == "stop"
    out = llm.generate([prompt], SamplingParams(max_new_tokens=10, ignore_eos=True))[0]
    assert out.token_ids == free and out.finish_reason == "length"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_starting_the_next_step_early_changes_nothing(gpu, dtype):
    """Requests that finish at different steps, by length and by the end token, greedy beside
    seeded temperature: the same tokens whether or not decode steps are started before the tokens
    of the step before have reached the host."""
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.TINY_B["vocab_size"]
    prompts = [util.rand_tokens(n, V, 70 + n) for n in (3, 17, 40, 9)]
    params = [SamplingParams(max_new_tokens=25), SamplingParams(temp=0.7, seed=3, max_new_tokens=40),
              SamplingParams(max_new_tokens=33), SamplingParams(temp=1.1, top_k=20, seed=4, max_new_tokens=12)]
    got = {}
    for ahead in (False, True):
        llm = LLM(util.model_folder("B", dtype), dtype=dtype, max_num_seqs=4, max_batched_tokens=32, ctx_size=128,
                  run_ahead=ahead)
        free = llm.generate(prompts, params)
        assert (llm.last_stats["steps_started_ahead"] > 20) == ahead
        llm.engine.model.eos_token_id = free[2].token_ids[10]         # request 2 stops early, the others go on
        stopped = llm.generate(prompts, params)
        assert stopped[2].finish_reason == "stop" and len(stopped[2].token_ids) <= 11
        got[ahead] = [o.token_ids for o in free] + [o.token_ids for o in stopped]
        llm.engine.manager.check()
        assert not llm.engine.manager.live()
    assert got[False] == got[True]


def _tuff(*args):
    return subprocess.run([sys.executable, os.path.join(util.ROOT, "bin", "tuff"), *args],
                          capture_output=True, text=True, timeout=300)


def test_command_line(gpu, tmp_path):
    folder = util.model_folder("A", "float32")
    prompt = util.rand_tokens(9, util.TINY_A["vocab_size"], 3)
    ids = ",".join(map(str, prompt))
    want, margins = plain_generate("A", prompt, 12, "float32")
    # --dump-tokens: ids on stdout, one a line
    p = _tuff("--model", folder, "--prompt-ids", ids, "--dump-tokens", "-n", "12", "--dtype", "fp32")
    assert p.returncode == 0, p.stderr
    got = [int(x) for x in p.stdout.split()]
    assert agree_up_to_near_ties(got, want, margins, 2e-5) == 12
    # prompt from a file, fed in portions of 4: same tokens
    f = tmp_path / "p.txt"
    f.write_text(" ".join(map(str, prompt)))
    p2 = _tuff("--model", folder, "--prompt-ids", str(f), "--dump-tokens", "-n", "12", "--dtype", "fp32", "--prefill-batch", "4")
    assert p2.returncode == 0 and p2.stdout == p.stdout
    # --teacher-force with --dump-logits: agreement 12/12 and the file holds the plain logits
    ref = tmp_path / "ref.txt"
    ref.write_text("\n".join(map(str, got)))
    out = tmp_path / "logits.bin"
    p3 = _tuff("--model", folder, "--prompt-ids", ids, "--teacher-force", str(ref), "--dump-logits", str(out),
               "--tf-batch", "4", "-n", "12", "--dtype", "fp32")
    assert p3.returncode == 0, p3.stderr
    assert "12/12" in p3.stderr
    raw = out.read_bytes()
    assert raw[:8] == b"CLBRLGT1"
    n, V = np.frombuffer(raw[8:16], dtype="<u4")
    assert (n, V) == (12, 512)
    rows = torch.from_numpy(np.frombuffer(raw[16:], dtype="<f4").reshape(12, 512).copy())
    full = util.plain_logits("A", prompt + got[:-1], "float32")[len(prompt) - 1:]
    util.assert_close_f32(rows, full, "teacher-forced logits")
    # a wrong reference is reported with exit code 1
    ref.write_text("\n".join(map(str, [got[0], (got[1] + 1) % 512] + got[2:])))
    p4 = _tuff("--model", folder, "--prompt-ids", ids, "--teacher-force", str(ref), "-n", "12", "--dtype", "fp32")
    assert p4.returncode == 1 and "top-1 agreement" in p4.stderr and "12/12" not in p4.stderr
    # timed mode prints the speed line; usage errors give 2; a broken model gives 1
    p5 = _tuff("--model", folder, "--prompt-ids", ids, "-n", "8", "--warmup", "2", "--runs", "2")
    assert p5.returncode == 0 and "Pipeline Generation Speed" in p5.stdout, p5.stderr
    assert "[Tuff timing]" not in p5.stderr
    # TUFF_TIMING=1: a line per phase on standard error, seconds since the mark before and since the start
    env = dict(os.environ, TUFF_TIMING="1")
    p6 = subprocess.run([sys.executable, os.path.join(util.ROOT, "bin", "tuff"), "--model", folder, "--prompt-ids", ids,
                         "-n", "4", "--warmup", "1", "--runs", "1"], capture_output=True, text=True, timeout=300, env=env)
    marks = [l for l in p6.stderr.splitlines() if l.startswith("[Tuff timing] ")]
    import re
    phases = [re.fullmatch(r"\[Tuff timing\] (.*): [0-9.]+ s \(t=[0-9.]+\)", m).group(1) for m in marks]
    assert p6.returncode == 0 and phases == ["config", "model_load", "run 0: prefill", "run 0: warmup", "run 0: decode"], \
        p6.stderr
    ts = [float(m.split("(t=")[1].rstrip(")")) for m in marks]
    assert ts == sorted(ts) and all(" s (t=" in m for m in marks)
    # bfloat16 (the default type), configuration B, whose greedy continuation is not one token repeated: the tokens of
    # the plain model up to its first near-tie, and teacher-forced on them the logits within the rounding model's noise
    folder16 = util.model_folder("B", "bfloat16")
    prompt16 = util.rand_tokens(11, util.TINY_B["vocab_size"], 5)
    ids16 = ",".join(map(str, prompt16))
    want16, margins16 = plain_generate("B", prompt16, 12, "bfloat16")
    p7 = _tuff("--model", folder16, "--prompt-ids", ids16, "--dump-tokens", "-n", "12")
    assert p7.returncode == 0, p7.stderr
    got16 = [int(x) for x in p7.stdout.split()]
    assert len(got16) == 12 and agree_up_to_near_ties(got16, want16, margins16, 2e-2) >= 1
    ref.write_text("\n".join(map(str, want16)))
    p8 = _tuff("--model", folder16, "--prompt-ids", ids16, "--teacher-force", str(ref), "--dump-logits", str(out),
               "--tf-batch", "5", "-n", "12", "--dtype", "bf16")
    assert p8.returncode in (0, 1), p8.stderr                 # 1: a first choice differs at a near-tie
    raw = out.read_bytes()
    n16, V16 = np.frombuffer(raw[8:16], dtype="<u4")
    assert (n16, V16) == (12, util.TINY_B["vocab_size"])
    rows16 = torch.from_numpy(np.frombuffer(raw[16:], dtype="<f4").reshape(12, V16).copy())
    util.assert_close("bfloat16", rows16, util.expected("B", prompt16 + want16[:-1], "bfloat16")[slice(len(prompt16) - 1, None)],
                      "teacher-forced logits, bfloat16")
    assert _tuff("--model", folder).returncode == 2
    assert _tuff("--model", folder, "--prompt-ids", ids, "-n", "5000").returncode == 2
    assert _tuff("--model", str(tmp_path), "--prompt-ids", ids).returncode == 1
    assert _tuff("--model", folder, "--inspect").returncode == 0


def test_gpu_time_by_kernel_class(gpu):
    """TUFF_TRACE=1: every entry point of the kernel libraries is timed with events and the run ends with a table of
    calls and GPU time by kernel class (the reference's TUFF_TRACE report, src/cupti_profiler.cu:115-181); the
    tokens are the same as without."""
    folder = util.model_folder("E", "bfloat16")
    ids = ",".join(map(str, util.rand_tokens(20, util.TINY_E["vocab_size"], 3)))
    plain_run = _tuff("--model", folder, "--prompt-ids", ids, "--dump-tokens", "-n", "6")
    env = dict(os.environ, TUFF_TRACE="1")
    p = subprocess.run([sys.executable, os.path.join(util.ROOT, "bin", "tuff"), "--model", folder, "--prompt-ids", ids,
                        "--dump-tokens", "-n", "6"], capture_output=True, text=True, timeout=300, env=env)
    assert p.returncode == 0, p.stderr
    assert p.stdout == plain_run.stdout and "GPU TIME BY KERNEL CLASS" not in plain_run.stderr
    assert "GPU TIME BY KERNEL CLASS" in p.stderr
    rows = {}
    for line in p.stderr.splitlines():
        cells = [c.strip() for c in line.split("|")]
        if len(cells) == 7 and cells[0].startswith("tuff_"):
            rows[cells[0]] = (int(cells[1]), float(cells[2]))
    # one prompt step and five steps of a single token through 2 attention layers, a head each step
    assert rows["tuff_attention_decode_fused"][0] == 10 and rows["tuff_attention_prefill"][0] == 2
    assert rows["tuff_embed_rows"][0] == 6 and all(ms > 0 for _, ms in rows.values())
    shares = [float(l.split("|")[6].strip().rstrip("%")) for l in p.stderr.splitlines() if l.startswith("tuff_") and l.count("|") == 6]
    assert abs(sum(shares) - 100) < 1.5


def test_command_line_jobs(gpu, tmp_path):
    """--jobs: the model is loaded once; every line is a run of its own with its own output files,
    exit code and environment (src/main.c:1921-2093)."""
    folder = util.model_folder("A", "float32")
    V = util.TINY_A["vocab_size"]
    a, b = util.rand_tokens(9, V, 3), util.rand_tokens(14, V, 4)
    ids = lambda p: ",".join(map(str, p))
    alone = [_tuff("--model", folder, "--dtype", "fp32", "--prompt-ids", ids(p), "--dump-tokens", "-n", "10").stdout
             for p in (a, b)]
    jobs = tmp_path / "jobs.txt"
    o = [tmp_path / f"o{i}" for i in range(4)]
    jobs.write_text(
        "# two runs, a usage error, and a run with an assignment in front\n"
        f"--prompt-ids {ids(a)} --dump-tokens -n 10 --out {o[0]} --err {tmp_path / 'e0'} --status {tmp_path / 's0'}\n"
        "\n"
        f"--prompt-ids '{' '.join(map(str, b))}' --dump-tokens -n 10 --out {o[1]}\n"
        f"--dump-tokens -n 10 --out {o[2]} --status {tmp_path / 's2'}\n"
        f"TUFF_TEST_MARK=1 --prompt-ids {ids(a)} --dump-tokens -n 10 --out {o[3]} --err {tmp_path / 'e3'}\n")
    p = _tuff("--model", folder, "--dtype", "fp32", "--jobs", str(jobs))
    assert p.returncode == 2, p.stderr                       # the first code that was not 0
    assert "4 job(s), 1 failed" in p.stderr
    said = p.stderr + (tmp_path / "e0").read_text() + (tmp_path / "e3").read_text()
    assert said.count("model ready") == 1 and said.count("reusing the loaded model") == 2      # job 3 never got that far
    assert o[0].read_text() == alone[0] and o[1].read_text() == alone[1] and o[3].read_text() == alone[0]
    assert (tmp_path / "s0").read_text().strip() == "0" and (tmp_path / "s2").read_text().strip() == "2"
    assert (tmp_path / "e0").read_text().strip().endswith("JOB_EXIT=0")
    assert "reusing the loaded model" in (tmp_path / "e3").read_text()
    assert "TUFF_TEST_MARK" not in os.environ


@pytest.mark.parametrize("name,seed", [("A", 3), ("B", 7), ("C", 18)])
def test_scheduler_scenarios_drawn_at_random(gpu, name, seed):
    """Requests, options, pool size, budget and slots drawn from a seed (greedy and seeded draws,
    repetition penalty, end tokens on and off, pools small enough to preempt, starting steps early
    on and off): in float32 every request generates what it generates alone."""
    import random
    from tuff_amd.engine.engine import Engine
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.CONFIGS[name][0]["vocab_size"]
    folder = util.model_folder(name, "float32")
    alone = LLM(engine=Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=256, max_requests=2),
                max_num_seqs=1, ctx_size=400)
    rng = random.Random(seed)
    n = rng.randint(3, 12)
    prompts = [util.rand_tokens(rng.randint(2, 90), V, seed * 100 + i) for i in range(n)]
    params = [SamplingParams(max_new_tokens=rng.randint(1, 40), ignore_eos=rng.random() < 0.7,
                             temp=rng.choice([0.0, 0.0, 0.8]), top_k=rng.choice([0, 20]), seed=rng.randint(1, 99),
                             repeat_penalty=rng.choice([1.0, 1.0, 1.2])) for _ in range(n)]
    pages = rng.randint(9, 30)
    llm = LLM(engine=Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=pages, max_requests=rng.randint(2, 5)),
              max_num_seqs=rng.randint(2, 5), max_batched_tokens=rng.choice([16, 48, 200]), ctx_size=400,
              run_ahead=rng.random() < 0.7)
    got = llm.generate(prompts, params)
    llm.engine.manager.check()
    assert not llm.engine.manager.live()
    for i, (p, sp, g) in enumerate(zip(prompts, params, got)):
        if g.finish_reason == "capacity":
            assert -(-(len(p) + sp.max_new_tokens) // 16) > pages
            continue
        want = alone.generate([p], sp)[0]
        assert (g.token_ids, g.finish_reason) == (want.token_ids, want.finish_reason), (seed, i, g.preemptions)


@pytest.mark.parametrize("name,seed", [("A", 2), ("C", 11)])
def test_scheduler_scenarios_with_steps_recorded_in_sections(gpu, name, seed):
    """The same with long prompts and a budget that is filled step after step, so that steps with
    portions are recorded and replayed (beside preemptions and steps started early): in float32
    every request still generates what it generates alone."""
    import random
    from tuff_amd.engine.engine import Engine
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    V = util.CONFIGS[name][0]["vocab_size"]
    folder = util.model_folder(name, "float32")
    alone = LLM(engine=Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=256, max_requests=2),
                max_num_seqs=1, ctx_size=1000)
    rng = random.Random(seed)
    n = rng.randint(4, 9)
    prompts = [util.rand_tokens(rng.randint(2, 700), V, seed * 100 + i) for i in range(n)]
    params = [SamplingParams(max_new_tokens=rng.randint(1, 40), ignore_eos=rng.random() < 0.7,
                             temp=rng.choice([0.0, 0.0, 0.8]), top_k=rng.choice([0, 20]), seed=rng.randint(1, 99))
              for _ in range(n)]
    pages = rng.randint(60, 120)
    llm = LLM(engine=Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=pages, max_requests=4),
              max_num_seqs=rng.randint(2, 4), max_batched_tokens=rng.choice([128, 130]), ctx_size=1000)
    got = llm.generate(prompts, params)
    llm.engine.manager.check()
    assert not llm.engine.manager.live() and llm.engine.section_replays >= 3
    for i, (p, sp, g) in enumerate(zip(prompts, params, got)):
        if g.finish_reason == "capacity":
            assert -(-(len(p) + sp.max_new_tokens) // 16) > pages
            continue
        want = alone.generate([p], sp)[0]
        assert (g.token_ids, g.finish_reason) == (want.token_ids, want.finish_reason), (seed, i, g.preemptions)
