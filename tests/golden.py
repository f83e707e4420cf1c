"""Frozen vectors of the engine's own float32 path: the sha256 of every logit row of fixed requests on the
tiny configurations, which every way of running them must reproduce byte for byte (whole, a head and single
tokens, changing portions, mixed with page reuse; recorded graphs on and off).  Within one run the tests
already demand that the cuttings agree with each other; the frozen vectors notice a change of the float32
arithmetic between two versions of the code (a sum in another order, a fused multiply-add more or less).

The method is the reference's (tools/lfm25_golden.py:118-248, tests/verify_lfm25_golden.sh:104-106,274-305:
a sha256 per teacher-forced logit row, an environment fingerprint, every configuration byte-identical,
updates only on purpose).  Its vectors themselves need its quantised checkpoint and cannot be used here.

A golden file is specific to what decides the bits: the GPU architecture and the compiler that built the
kernels (the fingerprint); where those differ the comparison says so instead of failing.  The model is named
by the sha256 of its model.safetensors, so a change of the random-weights generator shows as such.

    python tests/golden.py --check                       compare (needs the GPU)
    python tests/golden.py --update --reason "why"       write tests/golden/*.json anew, after checking that
                                                         all configurations of this run agree with each other
"""
from __future__ import annotations

import argparse
import datetime
import hashlib
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
GOLDEN_DIR = os.path.join(HERE, "golden")
FORMAT = 1
NAMES = ("A", "B")
LENGTHS = (45, 70, 33, 129)
PLANS = ("whole", "tail", "portions", "mixed")


def requests_for(name: str) -> dict:
    import util
    V = util.CONFIGS[name][0]["vocab_size"]
    return {f"g{i}": util.rand_tokens(n, V, 7000 + 10 * i + len(name)) for i, n in enumerate(LENGTHS)}


def plans_for(reqs: dict) -> dict:
    import util
    return {"whole": util.plan_whole(reqs), "tail": util.plan_tail(reqs, 32), "portions": util.plan_chunks(reqs),
            "mixed": util.plan_mixed(reqs, seed=11)}


def environment() -> dict:
    """What decides the bits of the float32 kernels (`fingerprint`) and what is recorded beside it."""
    import torch
    try:
        hipcc = subprocess.run(["hipcc", "--version"], capture_output=True, text=True).stdout
        hipcc = next((ln.strip() for ln in hipcc.splitlines() if "HIP version" in ln), hipcc.strip()[:80])
    except OSError:
        hipcc = "unknown"
    arch = torch.cuda.get_device_properties(0).gcnArchName.split(":")[0] if torch.cuda.is_available() else "no GPU"
    return {"fingerprint": {"gpu_arch": arch, "hipcc": hipcc},
            "torch": torch.__version__, "hip_runtime": getattr(torch.version, "hip", None)}


def model_identity(folder: str) -> dict:
    h = hashlib.sha256()
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        for block in iter(lambda: f.read(1 << 20), b""):
            h.update(block)
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return {"safetensors_sha256": h.hexdigest(), "config_sha256": hashlib.sha256(json.dumps(cfg, sort_keys=True).encode()).hexdigest()}


def row_hashes(logits) -> list[str]:
    """sha256 of every row's little-endian float32 bytes."""
    a = logits.detach().cpu().float().contiguous().numpy().astype("<f4")
    return [hashlib.sha256(a[i].tobytes()).hexdigest() for i in range(a.shape[0])]


def run_configuration(name: str, plan_name: str, use_graphs: bool) -> dict:
    """{request: (row hashes, first choices)} of one way of running the fixed requests in float32."""
    import util
    from tuff_amd.engine.engine import Engine
    reqs = requests_for(name)
    plan = plans_for(reqs)[plan_name]
    kw = dict(max_tokens=util.live_tokens_peak(plan), max_requests=4) if plan_name == "mixed" else dict(max_tokens=1024)
    eng = Engine.from_folder(util.model_folder(name, "bfloat16"), dtype="float32", page_size=16, poison_cache=True,
                             use_graphs=use_graphs, **kw)
    got = util.run_plan(eng, plan)
    return {rid: (row_hashes(got[rid]), [int(i) for i in got[rid].argmax(-1)]) for rid in reqs}


def configurations():
    return [(p, g) for p in PLANS for g in (True, False)]


def path_of(name: str) -> str:
    return os.path.join(GOLDEN_DIR, f"tiny_{name}_float32.json")


def compare(name: str, golden: dict, plan_name: str, use_graphs: bool) -> list[str]:
    """Messages about everything that differs from the golden in one configuration (none: byte-identical)."""
    got = run_configuration(name, plan_name, use_graphs)
    msgs = []
    for rid, g in golden["requests"].items():
        hashes, top1 = got[rid]
        if len(hashes) != len(g["row_sha256"]):
            msgs.append(f"{rid}: {len(hashes)} rows, golden {len(g['row_sha256'])}")
            continue
        bad = [i for i, (x, y) in enumerate(zip(hashes, g["row_sha256"])) if x != y]
        if bad:
            changed = sum(1 for i in bad if top1[i] != g["top1"][i])
            msgs.append(f"{rid}: first differing logit row {bad[0]}; differing rows {len(bad)}/{len(hashes)}; "
                        f"rows with another first choice {changed}")
    return msgs


def check_environment(name: str, golden: dict) -> list[str]:
    """Why the golden cannot be compared here (none: it can)."""
    import util
    bad = []
    if golden.get("format") != FORMAT:
        bad.append(f"format {golden.get('format')}, this program reads {FORMAT}")
    env = environment()
    for k, v in env["fingerprint"].items():
        if golden["environment"]["fingerprint"].get(k) != v:
            bad.append(f"environment.{k}: have {v!r}, golden {golden['environment']['fingerprint'].get(k)!r}")
    return bad


def check_model(name: str, golden: dict) -> list[str]:
    import util
    have = model_identity(util.model_folder(name, "bfloat16"))
    return [f"model {k}: have {v[:16]}.., golden {golden['model'].get(k, '')[:16]}.. (the random-weights generator or "
            f"the configuration has changed)" for k, v in have.items() if golden["model"].get(k) != v]


def update(reason: str, out_dir: str) -> int:
    import util
    os.makedirs(out_dir, exist_ok=True)
    for name in NAMES:
        runs = {c: run_configuration(name, *c) for c in configurations()}
        first_key = configurations()[0]
        first = runs[first_key]
        for c, got in runs.items():
            for rid in first:
                if got[rid][0] != first[rid][0]:
                    print(f"[golden] {name}: {c} and {first_key} differ on {rid}: nothing written", file=sys.stderr)
                    return 1
        try:
            commit = subprocess.run(["git", "rev-parse", "HEAD"], cwd=ROOT, capture_output=True, text=True).stdout.strip()
        except OSError:
            commit = ""
        reqs = requests_for(name)
        g = {"format": FORMAT, "configuration": name, "dtype": "float32",
             "model": model_identity(util.model_folder(name, "bfloat16")),
             "requests": {rid: {"tokens": len(reqs[rid]), "row_sha256": first[rid][0], "top1": first[rid][1]} for rid in reqs},
             "environment": environment(),
             "provenance": {"git_commit": commit, "reason": reason,
                            "date_utc": datetime.datetime.now(datetime.timezone.utc).strftime("%Y-%m-%dT%H:%M:%SZ"),
                            "configurations_verified_identical": [f"{p}/{'graphs' if gr else 'eager'}" for p, gr in configurations()]}}
        with open(os.path.join(out_dir, os.path.basename(path_of(name))), "w") as f:
            json.dump(g, f, indent=1)
            f.write("\n")
        print(f"[golden] {name}: {sum(len(v[0]) for v in first.values())} rows written, "
              f"{len(configurations())} configurations identical")
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--check", action="store_true")
    ap.add_argument("--update", action="store_true")
    ap.add_argument("--reason", default="")
    ap.add_argument("--out", default=GOLDEN_DIR, help="folder the golden files are written to")
    a = ap.parse_args(argv)
    sys.path.insert(0, ROOT)
    sys.path.insert(0, HERE)
    if a.update:
        if not a.reason:
            ap.error("--update needs --reason")
        return update(a.reason, a.out)
    bad = 0
    for name in NAMES:
        with open(path_of(name)) as f:
            golden = json.load(f)
        msgs = check_environment(name, golden) + check_model(name, golden)
        if msgs:
            print(f"[golden] {name}: not comparable here:\n    " + "\n    ".join(msgs))
            bad += 1
            continue
        for c in configurations():
            msgs = compare(name, golden, *c)
            print(f"[golden] {name} {c[0]}/{'graphs' if c[1] else 'eager'}: " + ("byte-identical" if not msgs else "FAIL"))
            for m in msgs:
                print("    " + m)
            bad += bool(msgs)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
