#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens a second of the LFM2.5-1.2B shape with random
weights (16 layers, 6 of them attention; hidden 2048), plus the 2,048-token prefill and decode at batch 1 and 64.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--layers L]

A "step" is one decode step of the whole batch through the serving loop (step function, greedy
pick on the GPU, the ids back on the host).  Every point is measured in RUNS runs of its own
(requests made and brought to their context anew); the value is the mean over the runs and `spread`
half the distance between the fastest and the slowest, as the reference reports its speeds
(src/main.c:1891-1904).  Prints one JSON line.

`probe` in that line is what this machine gives the product's own kernels where nothing but the memory
or the matrix cores bounds them (a product of 8 rows with 268 MB of weights, a product of 8192^3): the
denominators one may want beside the published peaks, which `roofline` and `frac` are priced against.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                                   # MI355X HBM3E, published
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}           # dense MFMA, published

# the config.json of the LFM2.5-1.2B shape
SHAPE = dict(
    architectures=["Lfm2ForCausalLM"], num_hidden_layers=16, full_attn_idxs=[2, 5, 8, 10, 12, 14],
    hidden_size=2048, num_attention_heads=32, num_key_value_heads=8, block_ff_dim=12288,
    block_auto_adjust_ff_dim=True, block_multiple_of=256, vocab_size=65536, rope_theta=1000000.0,
    conv_L_cache=3, norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=131072)
SEED = 2
LONG_POINTS = ((8, 32768), (1, 131072))                 # (batch, context) measured beside the benchmark's own context
PREFILL_TOKENS = 2048


def shape_config(layers: int):
    from tuff_amd.models.registry import config_from_dict
    raw = dict(SHAPE)
    if layers < raw["num_hidden_layers"]:
        raw["full_attn_idxs"] = [i for i in raw["full_attn_idxs"] if i < layers]
        raw["num_hidden_layers"] = layers
    return config_from_dict(raw)


def matmul_params(model) -> int:
    """Elements of all projection matrices of the layers (what the parts' Linear declare; not embedding,
    head, norms or conv taps)."""
    return sum(d.shape[0] * d.shape[1] for d in model.weight_decls() if d.role == "projection")


def prefill_flops(cfg, model, T: int, n_logits: int = 1) -> float:
    attn_layers = sum(1 for i in range(cfg.num_hidden_layers) if not cfg.is_conv(i))
    mm = 2.0 * matmul_params(model) * T
    attn = attn_layers * 2.0 * cfg.num_attention_heads * cfg.head_dim * T * T      # QK^T + PV, causal half
    head = 2.0 * cfg.vocab_size * cfg.hidden_size * n_logits
    return mm + attn + head


def decode_bytes(cfg, model, eng, batch: int, ctx: float) -> float:
    """Bytes a decode step has to read: every weight once, the cache of the live requests."""
    import torch
    elem = 2 if eng.dtype == torch.bfloat16 else 4
    weights = model.num_parameters() * elem
    kv = batch * ctx * eng.layout.bytes_per_token(elem)
    state = batch * eng.layout.state_bytes_per_request()
    return weights + kv + state


def run_decode(llm, cfg, batch: int, ctx_end: int, steps: int, warmup: int, seed: int):
    """`batch` requests are brought to ctx_end - steps - warmup tokens, then decoded; the last
    `steps` steps are timed.  Returns (seconds, mean context over the timed steps)."""
    import torch
    from tuff_amd.engine.batch import StepEntry
    from tuff_amd.engine.scheduler import Request
    from tuff_amd.sampling.params import SamplingParams
    g = torch.Generator().manual_seed(seed)
    eng = llm.engine
    # two tokens more than are timed: the loop starts a step before it has accounted for the one
    # before, so both time marks wait for a step that is already under way, and the window between
    # them holds exactly `steps` steps only if the run goes on past it
    n_new = steps + warmup + 2
    n_prompt = ctx_end - n_new
    sched = llm.new_scheduler()
    for b in range(batch):
        # the prompt but its last token goes through the step function in portions; the
        # scheduler takes the request over from there, so all requests decode together
        prompt = torch.randint(0, cfg.vocab_size, (n_prompt,), generator=g).tolist()
        rid = ("bench", batch, b)
        eng.begin(rid)
        for i in range(0, n_prompt - 1, PREFILL_TOKENS):
            eng.step([StepEntry(rid, prompt[i:min(i + PREFILL_TOKENS, n_prompt - 1)], [])])
        sched.adopt(Request(rid, prompt, SamplingParams(max_new_tokens=n_new, ignore_eos=True)), n_prompt - 1)
    marks = {}
    state = {"decode_steps": 0}

    def on_step(batch_, sampled):
        if all(len(s.tokens) == 1 for s in batch_) and len(batch_) == batch:
            state["decode_steps"] += 1
            if state["decode_steps"] == warmup:
                torch.cuda.synchronize()
                marks["t0"] = time.perf_counter()
            elif state["decode_steps"] == warmup + steps:
                torch.cuda.synchronize()
                marks["t1"] = time.perf_counter()
    llm.run(sched, on_step)
    if "t1" not in marks:
        raise RuntimeError(f"only {state['decode_steps']} pure decode steps ran; wanted {warmup + steps}")
    return marks["t1"] - marks["t0"], ctx_end - steps / 2.0


PREFILL_STREAM = 8               # prefill steps between two time marks


def run_prefill(llm, cfg, tokens: int, runs: int = 3, warmup: int = 4):
    """Prompts of `tokens` tokens, each in one step, to the first generated token.  Returns
    (seconds a step in a stream, seconds of a step from an idle GPU): the first as decode steps are
    timed, PREFILL_STREAM steps of as many requests between two synchronisations, `runs` times; the
    second one step at a time with the GPU idle before it (the host packs the step first, and the
    part's clocks take milliseconds to come back up), `PREFILL_STREAM` times.  Before either, `warmup`
    untimed steps (the engine records a step size that keeps coming when it comes for the third time;
    that one-off recording is not a prefill's time)."""
    import torch
    from tuff_amd.csrc import ops
    from tuff_amd.engine.batch import StepEntry
    eng = llm.engine
    g = torch.Generator().manual_seed(SEED + 1)
    picked = torch.empty(1, dtype=torch.int32, device=eng.device)
    count = [0]

    def stream(n: int) -> float:
        ids = [("prefill", count[0] + i) for i in range(n)]
        count[0] += n
        prompts = [torch.randint(0, cfg.vocab_size, (tokens,), generator=g).tolist() for _ in ids]
        for rid in ids:
            eng.begin(rid)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for rid, prompt in zip(ids, prompts):
            logits = eng.step([StepEntry(rid, prompt, [tokens - 1])])
            ops.argmax(logits, picked)
        int(picked.cpu()[0])                              # the last first token reaches the host
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        for rid in ids:
            eng.end(rid)
        return dt / n

    for _ in range(warmup):
        stream(1)
    stream(PREFILL_STREAM)                                # untimed: the stream's own warm-up
    in_stream = [stream(PREFILL_STREAM) for _ in range(runs)]
    alone = [stream(1) for _ in range(PREFILL_STREAM)]
    return in_stream, alone


def prefill_record(times, flops: float, dtype: str) -> dict:
    in_stream, alone = times
    dt, spread = mean_spread(in_stream)
    dt_alone, spread_alone = mean_spread(alone)
    return {"value": round(PREFILL_TOKENS / dt, 1), "tokens": PREFILL_TOKENS, "ms": round(dt * 1e3, 3),
            "frac": round(flops / dt / (PEAK_TFLOPS[dtype] * 1e12), 4), "runs": len(in_stream),
            "steps_a_run": PREFILL_STREAM, "spread_ms": round(spread * 1e3, 3),
            "from_idle_ms": round(dt_alone * 1e3, 3), "from_idle_spread_ms": round(spread_alone * 1e3, 3)}


LONG_PROMPT = 32768             # tokens of the long prompt point, fed in portions of PREFILL_TOKENS


def run_long_prompt(llm, cfg, tokens: int, runs: int = 3):
    """One prompt of `tokens` tokens through the step function in portions of PREFILL_TOKENS, to its
    first generated token.  Returns the seconds of `runs` runs after one untimed one."""
    import torch
    from tuff_amd.csrc import ops
    from tuff_amd.engine.batch import StepEntry
    eng = llm.engine
    g = torch.Generator().manual_seed(SEED + 7)
    picked = torch.empty(1, dtype=torch.int32, device=eng.device)
    times = []
    for run in range(runs + 1):
        prompt = torch.randint(0, cfg.vocab_size, (tokens,), generator=g).tolist()
        rid = ("long prompt", run)
        eng.begin(rid)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(0, tokens, PREFILL_TOKENS):
            part = prompt[i:i + PREFILL_TOKENS]
            last = i + PREFILL_TOKENS >= tokens
            logits = eng.step([StepEntry(rid, part, [len(part) - 1] if last else [])])
        ops.argmax(logits, picked)
        int(picked.cpu()[0])
        torch.cuda.synchronize()
        if run:
            times.append(time.perf_counter() - t0)
        eng.end(rid)
    return times


def mean_spread(values):
    return sum(values) / len(values), (max(values) - min(values)) / 2.0


def probe(device) -> dict:
    """What the machine gives the product's own kernels at their best shapes."""
    import torch
    from tuff_amd.csrc import ops
    g = torch.Generator(device=device).manual_seed(1)
    out = {}
    # read bandwidth: y = x W^T with 8 rows and 268 MB of weights, over four copies in turn (1 GB: more than any cache)
    N, K = 65536, 2048
    ws = [ops.tile_weight((torch.randn(N, K, generator=g, device=device) * 0.02).to(torch.bfloat16)) for _ in range(4)]
    x = torch.randn(8, K, generator=g, device=device).to(torch.bfloat16)
    y = torch.empty(8, N, dtype=torch.float32, device=device)
    for reps, keep in ((4, False), (40, True)):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(reps):
            ops.gemm(x, ws[i % 4], y)
        end.record()
        torch.cuda.synchronize()
        if keep:
            gbs = reps * N * K * 2 / (start.elapsed_time(end) * 1e-3) / 1e9
            out["read_GBs"] = round(gbs, 1)
            out["read_frac_of_published"] = round(gbs / HBM_PEAK_GBS, 4)
    del ws
    # matrix cores: a bfloat16 product of 8192^3
    n = 8192
    a = (torch.randn(n, n, generator=g, device=device) * 0.02).to(torch.bfloat16)
    w = ops.tile_weight((torch.randn(n, n, generator=g, device=device) * 0.02).to(torch.bfloat16))
    c = torch.empty(n, n, dtype=torch.bfloat16, device=device)
    for reps, keep in ((2, False), (10, True)):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            ops.gemm(a, w, c)
        end.record()
        torch.cuda.synchronize()
        if keep:
            tf = reps * 2.0 * n ** 3 / (start.elapsed_time(end) * 1e-3) / 1e12
            out["mfma_bf16_TFLOPs"] = round(tf, 1)
            out["mfma_frac_of_published"] = round(tf / PEAK_TFLOPS["bf16"], 4)
    return out


# Two serving runs through the scheduler, on other shapes of the architecture: many requests of very
# different lengths, prompts in portions beside decoding requests.
SCENARIOS = {
    "lfm2-2.6b": dict(
        config=dict(architectures=["Lfm2ForCausalLM"], num_hidden_layers=30,
                    full_attn_idxs=[2, 6, 10, 14, 18, 21, 24, 27], hidden_size=2048, num_attention_heads=32,
                    num_key_value_heads=8, block_ff_dim=16128, block_auto_adjust_ff_dim=True, block_multiple_of=256,
                    vocab_size=65536, rope_theta=1000000.0, conv_L_cache=3, norm_eps=1e-5, tie_word_embeddings=True,
                    max_position_embeddings=16384),
        seed=3, requests=32, at_a_time=32, budget=2048, new_tokens=256, prompts=("uniform", 128, 4096)),
    "lfm2-700m-long": dict(
        config=dict(architectures=["Lfm2ForCausalLM"], num_hidden_layers=16, full_attn_idxs=[2, 5, 8, 10, 12, 14],
                    hidden_size=1536, num_attention_heads=24, num_key_value_heads=8, block_ff_dim=6912,
                    block_auto_adjust_ff_dim=False, vocab_size=65536, rope_theta=1000000.0, conv_L_cache=3,
                    norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=32768),
        seed=4, requests=64, at_a_time=64, budget=512, new_tokens=64, prompts=("log-uniform", 16, 30000)),
}


def scenario_lengths(sc: dict) -> list:
    import math
    import random
    rng = random.Random(sc["seed"])
    kind, lo, hi = sc["prompts"]
    if kind == "uniform":
        return [rng.randint(lo, hi) for _ in range(sc["requests"])]
    return [int(math.exp(rng.uniform(math.log(lo), math.log(hi)))) for _ in range(sc["requests"])]


def scenario_pages(sc: dict) -> int:
    return sum(-(-(n + sc["new_tokens"]) // 16) for n in scenario_lengths(sc)) + 64


def run_scenario(name: str, dtype: str, runs: int = 3, eng=None) -> dict:
    """eng: an engine of the scenario's shape and seed with room for it (else one is made)."""
    import torch
    from tuff_amd.engine.engine import Engine
    from tuff_amd.engine.llm import LLM
    from tuff_amd.models.registry import config_from_dict
    from tuff_amd.sampling.params import SamplingParams
    sc = SCENARIOS[name]
    cfg = config_from_dict(sc["config"])
    lens = scenario_lengths(sc)
    new = sc["new_tokens"]
    if eng is None:
        eng = Engine.from_config(cfg, sc["seed"], dtype=dtype, page_size=16, num_pages=scenario_pages(sc),
                                 max_requests=sc["at_a_time"])
    llm = LLM(engine=eng, max_num_seqs=sc["at_a_time"], max_batched_tokens=sc["budget"],
              ctx_size=cfg.max_position_embeddings, ignore_eos=True)
    g = torch.Generator().manual_seed(SEED)
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lens]
    times = []
    for run in range(runs + 1):                            # the first run warms up
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = llm.generate(prompts, SamplingParams(max_new_tokens=new, ignore_eos=True))
        torch.cuda.synchronize()
        if run:
            times.append(time.perf_counter() - t0)
        if not all(len(o.token_ids) == new for o in outs):
            raise RuntimeError("a request of the scenario did not run to its end")
    total = sum(lens) + len(lens) * new
    st = llm.last_stats
    rate, spread = mean_spread([total / t for t in times])
    best = sum(times) / len(times)
    return {"metric": f"tokens/s through the scheduler, prompts and generated ({name})", "value": round(rate, 1),
            "unit": "tokens/s", "n_gpus": 1, "runs": len(times), "spread": round(spread, 1),
            "seconds": round(best, 3), "generated_per_s": round(len(lens) * new / best, 1),
            "dtype": dtype, "data": "synthetic: seeded random weights, uniform random token ids",
            "config": {"scenario": name, "requests": len(lens), "at_a_time": sc["at_a_time"], "prompt_tokens": sum(lens),
                       "longest_prompt": max(lens), "new_tokens_each": new, "max_batched_tokens": sc["budget"],
                       "layers": cfg.num_hidden_layers, "hidden": cfg.hidden_size, "ffn": cfg.ffn_dim,
                       "steps": st["steps"], "preemptions": st["preemptions"]}}


# Other shapes of the architecture, measured after the benchmark's own: decode at batch 8 and 64 at the benchmark's
# context, the 2,048-token prefill, and the shape's serving scenario on the same engine.
OTHER_SHAPES = {"2.6b": "lfm2-2.6b", "700m": "lfm2-700m-long"}           # key in `points` -> scenario whose config it is
FAR_BATCH, FAR_CONTEXT = 64, 32768                                         # attention is nine tenths of what this step reads
NEAR_CONTEXT = 256                                                         # ... and next to nothing of this one's


def describe_shape(cfg, model) -> str:
    return (f"{cfg.num_hidden_layers} layers (attention at {','.join(str(i) for i in cfg.full_attn_idxs)}), hidden {cfg.hidden_size}, "
            f"{cfg.num_attention_heads}/{cfg.num_key_value_heads} heads of {cfg.head_dim}, ffn {cfg.ffn_dim}, vocab {cfg.vocab_size}, "
            f"conv_L_cache {cfg.conv_L_cache}, {model.num_parameters()} parameters")


class Measured:
    """One engine of one shape and the points measured on it."""

    def __init__(self, cfg, seed: int, dtype: str, max_b: int, context: int, pages: int = 0, max_requests: int = 0):
        from tuff_amd.engine.engine import Engine
        from tuff_amd.engine.llm import LLM
        self.cfg, self.dtype, self.max_b, self.context, self.page = cfg, dtype, max_b, context, 16
        need = max(max_b * (-(-context // self.page)), PREFILL_STREAM * (PREFILL_TOKENS // self.page)) + PREFILL_TOKENS // self.page + 8
        self.eng = Engine.from_config(cfg, seed, dtype=dtype, page_size=self.page, num_pages=max(need, pages),
                                      max_requests=max(max_b, PREFILL_STREAM, max_requests) + 1)
        self.model = self.eng.model
        self.llm = LLM(engine=self.eng, max_num_seqs=max_b, max_batched_tokens=2048, ctx_size=context, ignore_eos=True)

    def tokens_of_room(self) -> int:
        return self.eng.manager.groups[0].pool.num_pages * self.page if self.eng.manager.groups else 0

    def decode_point(self, batch: int, steps: int, warmup: int, seed: int, runs: int, context: int = 0) -> dict:
        from tuff_amd.engine.llm import LLM
        context = context or self.context
        llm = self.llm
        if context != self.context:
            llm = LLM(engine=self.eng, max_num_seqs=self.max_b, max_batched_tokens=2048, ctx_size=context, ignore_eos=True)
        secs, ctx_mean = [], 0.0
        for run in range(runs):
            s_, ctx_mean = run_decode(llm, self.cfg, batch, context, steps, warmup, seed + 1000 * run)
            secs.append(s_)
        rate, spread = mean_spread([batch * steps / s_ for s_ in secs])
        step_s = sum(secs) / len(secs) / steps
        gbs = decode_bytes(self.cfg, self.model, self.eng, batch, ctx_mean) / step_s / 1e9
        return {"tok_s": rate, "spread": spread, "ms": 1e3 * step_s, "GBs": gbs}

    def prefill(self, runs: int, warmup: int) -> dict:
        flops = prefill_flops(self.cfg, self.model, PREFILL_TOKENS)
        return prefill_record(run_prefill(self.llm, self.cfg, PREFILL_TOKENS, runs=runs, warmup=warmup), flops, self.dtype)


def put(points: dict, key: str, pt: dict, spread: bool = False) -> None:
    points[key] = round(pt["tok_s"], 1)
    if spread:
        points[key + "_spread"] = round(pt["spread"], 1)
    points[key + "_ms_per_step"] = round(pt["ms"], 4)
    points[key + "_roofline_frac"] = round(pt["GBs"] / HBM_PEAK_GBS, 4)


def guarded(points: dict, key: str, fn) -> None:
    """A point beside the benchmark must not lose it: what fails is recorded in words."""
    try:
        fn()
    except Exception as e:                                    # noqa: BLE001
        points[key] = None
        points[key + "_error"] = f"{type(e).__name__}: {e}"[:200]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--no-long-points", dest="long_points", action="store_false",
                    help="skip the points further out: contexts of 256, 32768 and 131072, the long prompt")
    ap.add_argument("--no-other-shapes", dest="other_shapes", action="store_false",
                    help="skip the 2.6B and 700M shapes (decode at batch 8 and 64, prefill, their serving scenarios)")
    ap.add_argument("--layers", type=int, default=SHAPE["num_hidden_layers"],
                    help="fewer layers than the shape has (sizes of a layer stay)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip everything but the decode step at --batch")
    ap.add_argument("--point-steps", type=int, default=96)
    ap.add_argument("--runs", type=int, default=3, help="runs a point (mean and spread over them)")
    ap.add_argument("--no-probe", dest="probe", action="store_false",
                    help="skip the measurement of the machine's own read bandwidth and matrix rate")
    ap.add_argument("--prefill-warmup", type=int, default=4, help="untimed prefill runs before the timed ones")
    ap.add_argument("--only-prefill", action="store_true",
                    help="measure the 2,048-token prefill alone (for profiling) and print its record")
    ap.add_argument("--shape", default="1.2b", choices=["1.2b"] + sorted(OTHER_SHAPES),
                    help="measure another shape of the architecture in the benchmark's place (for profiling; "
                         "its points only, no other shapes after it)")
    ap.add_argument("--scenario", choices=sorted(SCENARIOS),
                    help="instead of the benchmark: a serving run through the scheduler on another shape")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; start it without a multi-process launcher")
        return 2

    if args.scenario:
        print(json.dumps(run_scenario(args.scenario, "bfloat16" if args.dtype == "bf16" else "float32", args.runs)))
        return 0

    import torch
    from tuff_amd.models.registry import config_from_dict

    cfg, seed, shape_name = shape_config(args.layers), SEED, "LFM2.5-1.2B"
    if args.shape != "1.2b":
        sc = SCENARIOS[OTHER_SHAPES[args.shape]]
        cfg, seed, shape_name = config_from_dict(sc["config"]), sc["seed"], OTHER_SHAPES[args.shape].upper().replace("-LONG", "")
        args.other_shapes = False
    max_b = args.batch if args.no_points else max(args.batch, 64)
    far = args.long_points and not args.no_points and args.dtype == "bf16"
    m = Measured(cfg, seed, args.dtype, max_b, args.context,
                 pages=(FAR_BATCH * FAR_CONTEXT // 16 + 64) if far else 0)
    eng, model = m.eng, m.model

    if args.only_prefill:
        print(json.dumps({"prefill": m.prefill(args.runs, args.prefill_warmup)}))
        return 0

    head = m.decode_point(args.batch, args.steps, args.warmup, seed, args.runs)
    further = []
    out = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} ({shape_name} shape)", "value": round(head["tok_s"], 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(head["ms"], 4),
        "runs": args.runs, "spread": round(head["spread"], 1),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": f"synthetic: seeded random weights (seed {seed}), uniform random token ids",
        "config": {
            "model": f"{shape_name} shape (Lfm2ForCausalLM)", "layers": cfg.num_hidden_layers,
            "layers_of_shape": SHAPE["num_hidden_layers"] if args.shape == "1.2b" else cfg.num_hidden_layers,
            "attention_layers": ",".join(str(i) for i in cfg.full_attn_idxs), "hidden": cfg.hidden_size,
            "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "ffn": cfg.ffn_dim, "vocab": cfg.vocab_size, "conv_L_cache": cfg.conv_L_cache,
            "tied_embeddings": cfg.tie_word_embeddings, "global_batch": args.batch, "seq_len": args.context,
            "parameters": model.num_parameters(),
            "constants": f"norm_eps {cfg.norm_eps}, rope_theta {cfg.rope_theta}, page_size {m.page}, prefill_tokens {PREFILL_TOKENS}",
            "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(head["GBs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(head["GBs"] / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        out["prefill"] = m.prefill(args.runs, args.prefill_warmup)
        points = {}
        for b in (1, 64):
            pt = m.decode_point(b, args.point_steps, 8, SEED + b, args.runs)
            put(points, f"decode_b{b}", pt, spread=True)
            points[f"decode_b{b}_GBs"] = round(pt["GBs"], 1)
        if args.long_points:
            room = m.tokens_of_room()

            def long_prompt():
                # a long prompt in portions: the attention over what earlier portions left is most of its work
                dt, spread = mean_spread(run_long_prompt(m.llm, cfg, LONG_PROMPT, args.runs))
                points[f"prompt_{LONG_PROMPT}_tok_s"] = round(LONG_PROMPT / dt, 1)
                points[f"prompt_{LONG_PROMPT}_ms"] = round(dt * 1e3, 2)
                points[f"prompt_{LONG_PROMPT}_spread_ms"] = round(spread * 1e3, 2)
            if LONG_PROMPT <= room:
                guarded(points, f"prompt_{LONG_PROMPT}_tok_s", long_prompt)
                further.append(f"a prompt of {LONG_PROMPT} in portions of {PREFILL_TOKENS}")
            # the same model nearer and further out: at a context of 256 a step reads weights and next to no cache
            # (the pure regime of few rows against a whole model), far out the cache is most of what it reads
            for b, ctx, steps, runs in ([(1, NEAR_CONTEXT, 64, args.runs), (8, NEAR_CONTEXT, 64, args.runs)]
                                        + [(b, ctx, 32, args.runs) for b, ctx in LONG_POINTS]
                                        + ([(FAR_BATCH, FAR_CONTEXT, 24, 1)] if far else [])):
                key = f"decode_b{b}_ctx{ctx}"
                if b * ctx > room or b > max_b:
                    continue                                  # the pool was made for less
                guarded(points, key, lambda: put(points, key, m.decode_point(b, steps, 4, SEED + ctx + b, runs, context=ctx)))
                further.append(f"decode b{b} ctx {ctx}" + (" (1 run)" if runs == 1 and args.runs != 1 else ""))
        out["points"] = points
    if args.probe and args.dtype == "bf16":
        del m.llm
        out["probe"] = probe(eng.device)
    if args.other_shapes and not args.no_points and args.dtype == "bf16" and args.layers == SHAPE["num_hidden_layers"]:
        del m, eng, model
        torch.cuda.empty_cache()
        for short, scenario in OTHER_SHAPES.items():
            sc = SCENARIOS[scenario]
            ocfg = config_from_dict(sc["config"])
            points = out["points"]

            def shape():
                o = Measured(ocfg, sc["seed"], args.dtype, 64, args.context, pages=scenario_pages(sc),
                             max_requests=sc["at_a_time"])
                out["config"][f"shape_{short}"] = describe_shape(ocfg, o.model) + f", seed {sc['seed']}"
                for b in (8, 64):
                    put(points, f"{short}_decode_b{b}", o.decode_point(b, 48, 8, sc["seed"] + b, 2 if b == 8 else 1))
                pre = o.prefill(2, args.prefill_warmup)
                points[f"{short}_prefill_tok_s"], points[f"{short}_prefill_ms"], points[f"{short}_prefill_frac"] = \
                    pre["value"], pre["ms"], pre["frac"]
                r = run_scenario(scenario, "bfloat16", 2, eng=o.eng)
                points[f"{short}_scenario_tok_s"], points[f"{short}_scenario_s"] = r["value"], r["seconds"]
                points[f"{short}_scenario_generated_per_s"] = r["generated_per_s"]
                del o
                torch.cuda.empty_cache()
            guarded(points, f"{short}_decode_b8", shape)
            c = sc["config"]
            kind, lo, hi = sc["prompts"]
            further.append(f"{short} shape: decode b8 (2 runs) and b64 (1 run) ctx {args.context}, prefill {PREFILL_TOKENS} (2 runs), scenario of "
                           f"{sc['requests']} requests with {kind} prompts of {lo} to {hi} tokens and {sc['new_tokens']} new each, "
                           f"{sc['budget']} tokens a step (2 runs after one)")
    if further:
        out["config"]["further_points"] = "; ".join(further)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
