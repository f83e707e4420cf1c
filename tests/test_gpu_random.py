"""Configurations and step plans drawn from seeds, against the plain implementation.

The fixed tiny configurations of the other tests differ in every size; here every size is drawn (head sizes
in steps of 8, heads and groups, widths and vocabularies that are no multiple of anything, two to six taps,
one to five layers of either kind in any order, page sizes), and so are the plans: portions of 1 to 200
tokens, any subset of places wanted (none too), requests that sit steps out, pools with no page to spare.
float32 must agree closely in every case.  In bfloat16 the conv mixers keep their quiet random weights: made loud
they amplify rounding, and single rows of single cases then pass any bound that a fault would still fail.
"""
import os
import random

import pytest
import torch

import util

pytestmark = pytest.mark.gpu


def random_plan(reqs: dict, rng: random.Random, max_live: int) -> list[dict]:
    waiting, live, steps = list(reqs.items()), {}, []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, end = [], []
        for rid, (toks, done) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.3:
                continue                                                   # sits this step out
            kind = rng.random()
            n = 1 if kind < 0.35 else rng.randint(2, 24) if kind < 0.7 else rng.randint(2, 200)
            n = min(n, len(toks) - done)
            w = rng.random()
            want = (list(range(n)) if w < 0.5 else [n - 1] if w < 0.7 else [] if w < 0.8
                    else sorted(rng.sample(range(n), rng.randint(1, n))))
            if done + n == len(toks):
                end.append(rid)
                if n - 1 not in want:
                    want = want + [n - 1]                                  # every request is looked at at least once
            entries.append({"id": rid, "tokens": toks[done:done + n], "want": want})
            live[rid][1] = done + n
        if not entries:
            continue
        for rid in end:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def pool_needed(plan, page_size: int) -> int:
    held, peak = {}, 0
    for s in plan:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-v // page_size) * page_size for v in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def check_wanted(plan, reqs, got, want_of, dtype, what):
    for rid, toks in reqs.items():
        wanted, pos = torch.zeros(len(toks), dtype=torch.bool), 0
        for s in plan:
            for e in s["entries"]:
                if e["id"] == rid:
                    wanted[[pos + w for w in e["want"]]] = True
                    pos += len(e["tokens"])
        assert torch.equal(~torch.isnan(got[rid]).all(-1), wanted), f"{what} {rid}: other rows than the wanted ones came back"
        util.assert_close(dtype, got[rid][wanted], want_of(rid)[wanted], f"{what} {rid}")


@pytest.mark.parametrize("seed", range(40))
def test_plans_drawn_at_random(gpu, seed):
    from tuff_amd.engine.engine import Engine
    rng = random.Random(1000 + seed)
    dtype = rng.choice(["float32", "bfloat16"])
    name = rng.choice(["A", "B", "C", "D", "E", "A+", "B+"])
    ps = rng.choice([16, 16, 32, 48, 64])
    V = util.CONFIGS[name.rstrip("+")][0]["vocab_size"]
    reqs = {f"r{i}": util.rand_tokens(rng.choice([rng.randint(2, 40), rng.randint(2, 330)]), V, seed * 100 + i)
            for i in range(rng.randint(1, 7))}
    plan = random_plan(reqs, rng, rng.randint(1, 4))
    eng = Engine.from_folder(util.model_folder(name, "bfloat16"), dtype=dtype, page_size=ps,
                             max_tokens=pool_needed(plan, ps), max_requests=4, poison_cache=True)
    got = util.run_plan(eng, plan)
    eng.manager.check()
    assert not eng.manager.live()
    check_wanted(plan, reqs, got, lambda rid: util.expected(name, reqs[rid], "bfloat16"), dtype,
                 f"seed {seed}: {name} {dtype} pages of {ps}")


@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random(gpu, seed, tmp_path):
    from plain.lfm2_plain import forward_logits, read_model
    from safetensors.torch import load_file, save_file
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models.registry import config_from_dict
    from tuff_amd.weights.random_init import write_random_model
    rng = random.Random(2000 + seed)
    hd = rng.choice([8, 16, 24, 32, 40, 48, 64, 64, 80, 96, 128])
    Hkv, G = rng.choice([1, 1, 2, 3, 4]), rng.choice([1, 2, 3, 4, 5, 8])
    while Hkv * G * hd > 768 and G > 1:
        G -= 1
    H = Hkv * G
    L = rng.randint(1, 5)
    types = [rng.choice(["conv", "full_attention"]) for _ in range(L)]
    auto = rng.random() < 0.4
    raw = dict(architectures=["Lfm2ForCausalLM"], num_hidden_layers=L, layer_types=types, hidden_size=H * hd,
               num_attention_heads=H, num_key_value_heads=Hkv,
               block_ff_dim=rng.choice([rng.randint(8, 64) * 8, rng.randint(3, 500)]), block_auto_adjust_ff_dim=auto,
               block_multiple_of=rng.choice([8, 32, 64, 256]), vocab_size=rng.randint(17, 3000),
               rope_theta=rng.choice([10000.0, 1e6, 5e5]), conv_L_cache=rng.randint(2, 6),
               norm_eps=rng.choice([1e-5, 1e-6, 3e-6, 1e-4]), tie_word_embeddings=rng.random() < 0.6,
               max_position_embeddings=4096)
    if auto and rng.random() < 0.5:
        raw["block_ffn_dim_multiplier"] = rng.choice([1.0, 1.3, 0.7])
    dtype = rng.choice(["float32", "bfloat16"])
    ps = rng.choice([16, 16, 32, 64])
    folder = str(tmp_path / "model")
    write_random_model(config_from_dict(raw), folder, seed, torch.bfloat16)
    if rng.random() < 0.5:                                                 # loud conv mixers
        path = os.path.join(folder, "model.safetensors")
        tensors = load_file(path)
        for k in tensors:
            for suffix, factor in util.LOUD_CONV.items():
                if k.endswith(suffix):
                    tensors[k] = (tensors[k].float() * factor).to(tensors[k].dtype)
        save_file(tensors, path)
    eng = Engine.from_folder(folder, dtype=dtype, page_size=ps, max_tokens=1024, max_requests=4, poison_cache=True)
    V = raw["vocab_size"]
    reqs = {f"r{i}": util.rand_tokens(rng.choice([rng.randint(2, 40), rng.randint(41, 300)]), V, seed * 10 + i) for i in range(3)}
    pcfg, pw = read_model(folder)
    want = {rid: util.expected_of(pcfg, pw, t) for rid, t in reqs.items()}
    what = f"seed {seed}: {dtype} pages of {ps}, {H} heads of {hd} on {Hkv}, layers {''.join(t[0] for t in types)}"
    for pname, plan in (("whole", util.plan_whole(reqs)), ("tail", util.plan_tail(reqs, 12)), ("portions", util.plan_chunks(reqs)),
                        ("mixed", util.plan_mixed(reqs, seed=seed)), ("random", random_plan(reqs, rng, 3))):
        got = util.run_plan(eng, plan)
        eng.manager.check()
        check_wanted(plan, reqs, got, lambda rid: want[rid], dtype, f"{what}, {pname}")
