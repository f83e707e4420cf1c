#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens a second of the LFM2.5-1.2B shape with random
weights (16 layers, 6 of them attention; hidden 2048), plus the 2,048-token prefill and decode at batch 1 and 64.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--layers L]

A "step" is one decode step of the whole batch through the serving loop (step function, greedy
pick on the GPU, the ids back on the host).  Prints one JSON line.
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
    conv_L_cache=3, norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=8192)
SEED = 2
PREFILL_TOKENS = 2048


def shape_config(layers: int):
    from tuff_amd.models.registry import config_from_dict
    raw = dict(SHAPE)
    if layers < raw["num_hidden_layers"]:
        raw["full_attn_idxs"] = [i for i in raw["full_attn_idxs"] if i < layers]
        raw["num_hidden_layers"] = layers
    return config_from_dict(raw)


def matmul_params(model) -> int:
    """Elements of all projection matrices of the layers (not embedding, head or norms)."""
    skip = {model.embedding_decl.name} | ({model.head_decl.name} if model.head_decl else set())
    return sum(d.shape[0] * d.shape[1] for d in model.weight_decls()
               if len(d.shape) == 2 and d.name not in skip and d.init == "normal" and d.shape[1] > 16)


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


def run_prefill(llm, cfg, tokens: int, repeats: int = 8):
    import torch
    from tuff_amd.csrc import ops
    from tuff_amd.engine.batch import StepEntry
    eng = llm.engine
    g = torch.Generator().manual_seed(SEED + 1)
    best = None
    picked = torch.empty(1, dtype=torch.int32, device=eng.device)
    for i in range(repeats + 1):
        prompt = torch.randint(0, cfg.vocab_size, (tokens,), generator=g).tolist()
        eng.begin(("prefill", i))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = eng.step([StepEntry(("prefill", i), prompt, [tokens - 1])])
        ops.argmax(logits, picked)
        nxt = int(picked.cpu()[0])                        # the first generated token reaches the host
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        eng.end(("prefill", i))
        if i > 0:                                         # the first run warms up; the best of the rest counts
            best = dt if best is None else min(best, dt)
    return best


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


def run_scenario(name: str, dtype: str) -> dict:
    import math
    import random
    import torch
    from tuff_amd.engine.engine import Engine
    from tuff_amd.engine.llm import LLM
    from tuff_amd.models.registry import config_from_dict
    from tuff_amd.sampling.params import SamplingParams
    sc = SCENARIOS[name]
    cfg = config_from_dict(sc["config"])
    rng = random.Random(sc["seed"])
    kind, lo, hi = sc["prompts"]
    if kind == "uniform":
        lens = [rng.randint(lo, hi) for _ in range(sc["requests"])]
    else:
        lens = [int(math.exp(rng.uniform(math.log(lo), math.log(hi)))) for _ in range(sc["requests"])]
    new = sc["new_tokens"]
    pages = sum(-(-(n + new) // 16) for n in lens) + 64
    eng = Engine.from_config(cfg, sc["seed"], dtype=dtype, page_size=16, num_pages=pages, max_requests=sc["at_a_time"])
    llm = LLM(engine=eng, max_num_seqs=sc["at_a_time"], max_batched_tokens=sc["budget"],
              ctx_size=cfg.max_position_embeddings, ignore_eos=True)
    g = torch.Generator().manual_seed(SEED)
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lens]
    best = None
    for _ in range(2):                                     # the first run warms up
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = llm.generate(prompts, SamplingParams(max_new_tokens=new, ignore_eos=True))
        torch.cuda.synchronize()
        best = time.perf_counter() - t0
        if not all(len(o.token_ids) == new for o in outs):
            raise RuntimeError("a request of the scenario did not run to its end")
    total = sum(lens) + len(lens) * new
    st = llm.last_stats
    return {"metric": f"tokens/s through the scheduler, prompts and generated ({name})", "value": round(total / best, 1),
            "unit": "tokens/s", "n_gpus": 1, "seconds": round(best, 3), "generated_per_s": round(len(lens) * new / best, 1),
            "dtype": dtype, "data": "synthetic: seeded random weights, uniform random token ids",
            "config": {"scenario": name, "requests": len(lens), "at_a_time": sc["at_a_time"], "prompt_tokens": sum(lens),
                       "longest_prompt": max(lens), "new_tokens_each": new, "max_batched_tokens": sc["budget"],
                       "layers": cfg.num_hidden_layers, "hidden": cfg.hidden_size, "ffn": cfg.ffn_dim,
                       "steps": st["steps"], "preemptions": st["preemptions"]}}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=SHAPE["max_position_embeddings"])
    ap.add_argument("--layers", type=int, default=SHAPE["num_hidden_layers"],
                    help="fewer layers than the shape has (sizes of a layer stay)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip prefill and the batch 1 / 64 points")
    ap.add_argument("--point-steps", type=int, default=96)
    ap.add_argument("--only-prefill", action="store_true",
                    help="measure the 2,048-token prefill alone (for profiling) and print its record")
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
        print(json.dumps(run_scenario(args.scenario, "bfloat16" if args.dtype == "bf16" else "float32")))
        return 0

    import torch
    from tuff_amd.engine.engine import Engine
    from tuff_amd.engine.llm import LLM

    cfg = shape_config(args.layers)
    page = 16
    max_b = args.batch if args.no_points else max(args.batch, 64)
    pages = max_b * (-(-args.context // page)) + PREFILL_TOKENS // page + 8
    eng = Engine.from_config(cfg, SEED, dtype=args.dtype, page_size=page, num_pages=pages, max_requests=max_b + 1)
    llm = LLM(engine=eng, max_num_seqs=max_b, max_batched_tokens=2048, ctx_size=args.context, ignore_eos=True)
    model = eng.model

    if args.only_prefill:
        dt = run_prefill(llm, cfg, PREFILL_TOKENS)
        flops = prefill_flops(cfg, model, PREFILL_TOKENS)
        print(json.dumps({"prefill": {"value": round(PREFILL_TOKENS / dt, 1), "tokens": PREFILL_TOKENS,
                                      "ms": round(dt * 1e3, 3),
                                      "frac": round(flops / dt / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}}))
        return 0
    secs, ctx_mean = run_decode(llm, cfg, args.batch, args.context, args.steps, args.warmup, SEED)
    tok_s = args.batch * args.steps / secs
    ms_step = 1e3 * secs / args.steps
    achieved = decode_bytes(cfg, model, eng, args.batch, ctx_mean) / (secs / args.steps) / 1e9
    out = {
        "metric": "decode tok/s at batch 8, context 8192 (LFM2.5-1.2B shape)", "value": round(tok_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: seeded random weights (seed 2), uniform random token ids",
        "config": {
            "model": "LFM2.5-1.2B shape (Lfm2ForCausalLM)", "layers": cfg.num_hidden_layers,
            "layers_of_shape": SHAPE["num_hidden_layers"],
            "attention_layers": ",".join(str(i) for i in cfg.full_attn_idxs), "hidden": cfg.hidden_size,
            "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "ffn": cfg.ffn_dim, "vocab": cfg.vocab_size, "conv_L_cache": cfg.conv_L_cache,
            "tied_embeddings": cfg.tie_word_embeddings, "global_batch": args.batch, "seq_len": args.context,
            "prefill_tokens": PREFILL_TOKENS, "page_size": page, "parameters": model.num_parameters(),
            "norm_eps": cfg.norm_eps, "rope_theta": cfg.rope_theta,
            "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        dt = run_prefill(llm, cfg, PREFILL_TOKENS)
        flops = prefill_flops(cfg, model, PREFILL_TOKENS)
        out["prefill"] = {"value": round(PREFILL_TOKENS / dt, 1), "tokens": PREFILL_TOKENS, "ms": round(dt * 1e3, 3),
                          "frac": round(flops / dt / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}
        points = {}
        for b in (1, 64):
            s, _ = run_decode(llm, cfg, b, args.context, args.point_steps, 8, SEED + b)
            points[f"decode_b{b}"] = round(b * args.point_steps / s, 1)
        out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
