"""Command line in the manner of the reference's `tuff` (src/main.c:45-97, :769-979): the same
option names and meanings where it has them, ids instead of text where a random model has no
vocabulary.

    tuff --model DIR --prompt-ids 1,36309 -n 128 [--temp 0.8 --seed 7 ...]
    tuff --model DIR --prompt-ids p.txt --dump-tokens -n 32
    tuff --model DIR --prompt-ids p.txt --teacher-force ref.txt --dump-logits out.bin --tf-batch 4
    tuff --random config.json --seed 2 --inspect
    tuff --model DIR --jobs jobs.txt            (the model is loaded once, every line is a run)

Exit codes as in the reference: 0 ok, 1 mismatch or model error, 2 usage, 3 engine or IO failure.
"""
from __future__ import annotations

import argparse
import json
import os
import struct
import sys
import tempfile
import time


def _ids_from(text_or_path: str) -> list[int]:
    src = text_or_path
    if os.path.isfile(src):
        with open(src) as f:
            src = f.read()
    return [int(t) for t in src.replace(",", " ").split()]


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="tuff", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter,
                                 epilog="Environment: TUFF_TIMING=1 prints one line per phase (configuration, model load, "
                                        "prefill, warm-up, decode) with its seconds on standard error.  TUFF_TRACE=1 "
                                        "times every class of kernels with events (no recorded graphs meanwhile) and "
                                        "prints a table of GPU time by kernel class at the end of the run.")
    ap.add_argument("--model", help="model folder (config.json + model.safetensors)")
    ap.add_argument("--random", metavar="CONFIG_JSON", help="random weights for this config.json instead of --model")
    ap.add_argument("--prompt", "-p", help="prompt text (needs tokenizer.json in the model folder)")
    ap.add_argument("--prompt-file", help="read the prompt text from a file")
    ap.add_argument("--prompt-ids", help="prompt as token ids: a file or a comma/space separated list")
    ap.add_argument("-c", "--ctx-size", "--max-seq", "--ctx", "--context-size", dest="ctx", type=int, default=4096,
                    help="maximum context sequence length (default: 4096)")
    ap.add_argument("-n", dest="n_predict", type=int, default=None, help="tokens to generate (default: 128; 32 in dump modes)")
    ap.add_argument("--warmup", type=int, default=32, help="warm-up tokens before the timed ones (default: 32)")
    ap.add_argument("--runs", type=int, default=3, help="benchmark runs (default: 3)")
    ap.add_argument("--prefill-batch", type=int, default=None,
                    help="feed the prompt in portions of N tokens (default: --max-batched-tokens)")
    ap.add_argument("--tf-batch", type=int, default=1, help="with --teacher-force: feed the reference in chunks of B tokens")
    ap.add_argument("--inspect", action="store_true", help="print the model inventory and exit")
    ap.add_argument("--dump-tokens", action="store_true", help="print generated token ids to stdout, one a line")
    ap.add_argument("--dump-logits", metavar="PATH", help="dump the logit vector of every step")
    ap.add_argument("--teacher-force", metavar="FILE", help="feed reference token ids, report per-step top-1 agreement")
    ap.add_argument("--temp", "--temperature", dest="temp", type=float, default=0.0)
    ap.add_argument("--top-p", "--top_p", dest="top_p", type=float, default=1.0)
    ap.add_argument("--top-k", "--top_k", dest="top_k", type=int, default=0)
    ap.add_argument("--min-p", "--min_p", dest="min_p", type=float, default=0.0)
    ap.add_argument("--repeat-penalty", "--repeat_penalty", dest="repeat_penalty", type=float, default=1.0)
    ap.add_argument("--repeat-last-n", "--repeat_last_n", dest="repeat_last_n", type=int, default=64)
    ap.add_argument("--seed", type=int, default=0, help="sampling seed (0: from the clock); weights seed with --random")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "bfloat16", "fp32", "float32"])
    ap.add_argument("--max-num-seqs", type=int, default=8)
    ap.add_argument("--max-batched-tokens", type=int, default=2048)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=None)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--jobs", metavar="FILE", help="one job a line: [NAME=value ...] <tuff arguments> [--out F] [--err F] "
                                                    "[--status F]; the model is loaded once")
    ap.add_argument("--out", help="in a job: the job's standard output goes to this file")
    ap.add_argument("--err", help="in a job: the job's standard error goes to this file")
    ap.add_argument("--status", help="in a job: the job's exit code is written to this file")
    return ap


def _inspect(cfg, model, out=sys.stdout) -> None:
    """Inventory in the spirit of lfm25_model_print_inspection (src/lfm25_model.c:381-401)."""
    print(f"architecture: {cfg.architecture}", file=out)
    for k, v in cfg.to_dict().items():
        if k != "architectures":
            print(f"  {k}: {v}", file=out)
    n = model.num_parameters()
    print(f"parameters: {n} ({2 * n / 2**20:.1f} MiB in bfloat16)", file=out)
    for i, b in enumerate(model.blocks):
        # a block of another arrangement may have neither a mixer nor a feed-forward of these names
        mixer, ffn = getattr(b, "mixer", None), getattr(b, "ffn", None)
        inside = " + ".join(type(p).__name__ for p in (mixer, ffn) if p is not None) or type(b).__name__
        spec = mixer.cache_spec() if hasattr(mixer, "cache_spec") else None
        print(f"  layer {i}: {inside}  cache: {spec}", file=out)
    print(f"run order: {[r.block for r in model.schedule]}", file=out)


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if "--jobs" in argv:
        return _run_jobs(argv)
    return _run(argv, {})


def _run_jobs(argv: list) -> int:
    """`--jobs FILE` as in the reference (src/main.c:1921-2093): one process, one model load, many
    jobs.  A job's command line is this invocation's arguments (without --jobs) followed by the
    line's; leading NAME=value tokens are its environment (restored afterwards); --out/--err take its
    output, the last line of its standard error is JOB_EXIT=<code>, --status gets the code.  Blank
    lines and lines starting with '#' are skipped.  Returns 0 if every job did, else the first
    job's code that was not 0."""
    import contextlib
    import shlex
    i = argv.index("--jobs")
    if i + 1 >= len(argv):
        print("tuff: --jobs needs a file", file=sys.stderr)
        return 2
    path, defaults = argv[i + 1], argv[:i] + argv[i + 2:]
    try:
        with open(path) as f:
            lines = f.readlines()
    except OSError as e:
        print(f"tuff: cannot open the jobs file: {e}", file=sys.stderr)
        return 2
    loaded: dict = {}
    overall = njob = nfail = 0
    for line in lines:
        if not line.strip() or line.lstrip().startswith("#"):
            continue
        njob += 1
        rc, env, job_args = 0, {}, []
        try:
            tokens = shlex.split(line)
        except ValueError as e:
            print(f"tuff: jobs: line {njob}: {e}", file=sys.stderr)
            tokens, rc = [], 2
        while tokens and "=" in tokens[0] and (tokens[0][0].isalpha() or tokens[0][0] == "_") \
                and tokens[0].split("=", 1)[0].replace("_", "a").isalnum():
            name, value = tokens.pop(0).split("=", 1)
            env[name] = value
        job_args = defaults + tokens

        def last(opt):
            hits = [k for k in range(len(job_args) - 1) if job_args[k] == opt]
            return job_args[hits[-1] + 1] if hits else None
        out_path, err_path, status_path = last("--out"), last("--err"), last("--status")
        saved = {k: os.environ.get(k) for k in env}
        os.environ.update(env)
        with contextlib.ExitStack() as stack:
            fo = stack.enter_context(open(out_path, "w")) if out_path else None
            fe = stack.enter_context(open(err_path, "w")) if err_path else None
            if fo:
                stack.enter_context(contextlib.redirect_stdout(fo))
            if fe:
                stack.enter_context(contextlib.redirect_stderr(fe))
            if rc == 0:
                try:
                    rc = _run(job_args, loaded)
                except Exception as e:                       # noqa: BLE001 - a job must not take the runner down
                    print(f"tuff: {type(e).__name__}: {e}", file=sys.stderr)
                    rc = 3
            sys.stdout.flush()
            print(f"JOB_EXIT={rc}", file=sys.stderr)
            sys.stderr.flush()
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        if status_path:
            with open(status_path, "w") as f:
                f.write(f"{rc}\n")
        print(f"tuff: job {njob}: exit {rc}" + (f" err={err_path}" if err_path else ""), file=sys.stderr)
        if rc != 0:
            nfail += 1
            overall = overall or rc
    print(f"tuff: jobs: {njob} job(s), {nfail} failed", file=sys.stderr)
    return overall


class _Timing:
    """TUFF_TIMING=1: one line per phase on stderr, "[Tuff timing] <phase>: <seconds since the mark
    before> s (t=<seconds since the run began>)", as the reference prints them (src/main.c:204-225).
    A mark waits for the GPU first, so a phase's time holds the work it started."""

    def __init__(self):
        self.on = os.environ.get("TUFF_TIMING", "")[:1] == "1"
        self.start = self.last = time.monotonic()

    def mark(self, what: str, sync: bool = True) -> None:
        if not self.on:
            return
        if sync:
            try:
                import torch
                if torch.cuda.is_available():
                    torch.cuda.synchronize()
            except Exception:                                # noqa: BLE001 - a mark never ends a run
                pass
        now = time.monotonic()
        print(f"[Tuff timing] {what}: {now - self.last:.3f} s (t={now - self.start:.3f})", file=sys.stderr)
        self.last = now


def _run(argv: list, loaded: dict) -> int:
    """One run.  `loaded` keeps the engine from one run of a job file to the next."""
    tm = _Timing()
    ap = build_parser()
    try:
        args = ap.parse_args(argv)
    except SystemExit as e:
        return 2 if e.code not in (0, None) else 0
    if bool(args.model) == bool(args.random):
        print("tuff: give exactly one of --model and --random", file=sys.stderr)
        return 2
    from .config.base import ConfigError
    from .models.registry import build_model, config_from_dict, load_config
    try:
        if args.random:
            with open(args.random) as f:
                cfg = config_from_dict(json.load(f))
        else:
            cfg = load_config(args.model)
    except (ConfigError, OSError, json.JSONDecodeError) as e:
        print(f"tuff: {e}", file=sys.stderr)
        return 1
    tm.mark("config", sync=False)
    if args.inspect:
        _inspect(cfg, build_model(cfg))
        return 0

    # ---- prompt
    ids = None
    if args.prompt_ids is not None:
        try:
            ids = _ids_from(args.prompt_ids)
        except ValueError as e:
            print(f"tuff: --prompt-ids: {e}", file=sys.stderr)
            return 2
    elif args.prompt is not None or args.prompt_file is not None:
        text = args.prompt
        if args.prompt_file:
            try:
                with open(args.prompt_file, encoding="utf-8") as f:
                    text = f.read()
            except OSError as e:
                print(f"tuff: {e}", file=sys.stderr)
                return 2
        tok_path = os.path.join(args.model or "", "tokenizer.json")
        if not os.path.isfile(tok_path):
            print("tuff: --prompt needs tokenizer.json in the model folder; use --prompt-ids", file=sys.stderr)
            return 2
        from tokenizers import Tokenizer
        ids = Tokenizer.from_file(tok_path).encode(text).ids
    if not ids:
        print("tuff: no prompt: give --prompt-ids (or --prompt with a tokenizer)", file=sys.stderr)
        return 2

    dump_mode = args.dump_tokens or args.dump_logits or args.teacher_force
    n_predict = args.n_predict if args.n_predict is not None else (32 if dump_mode else 128)
    chunk = args.prefill_batch or args.max_batched_tokens

    # ---- engine
    try:
        from .engine.engine import Engine
        from .engine.llm import LLM
        from .engine.batch import StepEntry
        from .sampling.params import SamplingParams
        ctx = min(args.ctx, getattr(cfg, "max_position_embeddings", args.ctx))
        pages = args.num_pages or args.max_num_seqs * -(-ctx // args.page_size)
        kw = dict(dtype=args.dtype, page_size=args.page_size, num_pages=pages, max_requests=args.max_num_seqs)
        key = (os.path.abspath(args.random or args.model), bool(args.random), args.seed if args.random else None,
               tuple(sorted(kw.items())))
        if loaded.get("key") == key:
            eng = loaded["engine"]
            for rid in eng.manager.live():                   # a run that failed may have left requests behind
                eng.end(rid)
            print(f"tuff: jobs: reusing the loaded model {args.random or args.model}", file=sys.stderr)
        else:
            loaded.clear()
            t0 = time.time()
            if args.random:
                eng = Engine.from_config(cfg, args.seed, **kw)
            else:
                eng = Engine.from_folder(args.model, **kw)
            loaded.update(key=key, engine=eng)
            print(f"tuff: model ready in {time.time() - t0:.2f} s", file=sys.stderr)
        tm.mark("model_load")
    except Exception as e:                                   # noqa: BLE001 - reported, then exit code
        print(f"tuff: {type(e).__name__}: {e}", file=sys.stderr)
        return 1 if type(e).__name__ in ("WeightsError", "ConfigError") else 3
    llm = LLM(engine=eng, max_num_seqs=args.max_num_seqs, max_batched_tokens=chunk, ctx_size=ctx,
              ignore_eos=args.ignore_eos or bool(dump_mode) or args.n_predict is not None)
    params = SamplingParams(temp=args.temp, top_p=args.top_p, top_k=args.top_k, min_p=args.min_p,
                            repeat_penalty=args.repeat_penalty, repeat_last_n=args.repeat_last_n,
                            seed=args.seed, max_new_tokens=n_predict, ignore_eos=True)
    if len(ids) + n_predict > ctx:
        print(f"tuff: prompt ({len(ids)}) + -n ({n_predict}) does not fit -c {ctx}", file=sys.stderr)
        return 2

    from .csrc import ops
    if ops.TRACE:
        ops.trace_reset()                                    # the model's loading is not part of the run
    try:
        if args.teacher_force or args.dump_logits:
            rc = _teacher_force(args, eng, ids, n_predict, chunk)
            tm.mark("teacher_force")
            return rc
        if args.dump_tokens:
            out = llm.generate([ids], params)[0]
            tm.mark("generate")
            for t in out.token_ids:
                print(t)
            print(f"tuff: {len(out.token_ids)} tokens, finish: {out.finish_reason}", file=sys.stderr)
            return 0
        return _timed(args, llm, ids, params, tm)
    except Exception as e:                                   # noqa: BLE001
        print(f"tuff: {type(e).__name__}: {e}", file=sys.stderr)
        return 3
    finally:
        if ops.TRACE:
            ops.trace_report(sys.stderr)


def _timed(args, llm, ids, params, tm) -> int:
    """Warm-up then timed decode, mean +- (max - min)/2 over runs (src/main.c:1720-1726, :1891-1904)."""
    import dataclasses
    import torch
    from .engine.scheduler import Request
    rates, last = [], None
    for run in range(max(1, args.runs)):
        sched = llm.new_scheduler()
        p = dataclasses.replace(params, max_new_tokens=params.max_new_tokens + args.warmup)
        req = Request(("run", run), list(ids), p)
        sched.add(req)
        marks = {}

        def on_step(batch, sampled, req=req, marks=marks, run=run):
            n = len(req.output)
            if n >= 1 and "prefill" not in marks:
                torch.cuda.synchronize()
                marks["prefill"] = time.perf_counter()
                tm.mark(f"run {run}: prefill", sync=False)
            if n >= args.warmup + 1 and "t0" not in marks:
                torch.cuda.synchronize()
                marks["t0"] = time.perf_counter()
                tm.mark(f"run {run}: warmup", sync=False)
        torch.cuda.synchronize()
        t_start = time.perf_counter()
        llm.run(sched, on_step)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        tm.mark(f"run {run}: decode", sync=False)
        timed = len(req.output) - args.warmup - 1
        if timed > 0 and "t0" in marks:
            rates.append(timed / (t1 - marks["t0"]))
        if "prefill" in marks:
            print(f"tuff: run {run}: prefill {len(ids)} tokens in {(marks['prefill'] - t_start) * 1e3:.1f} ms "
                  f"({len(ids) / (marks['prefill'] - t_start):.0f} tok/s)", file=sys.stderr)
        last = req
    if last is not None:
        print(" ".join(str(t) for t in last.output[:16]) + (" ..." if len(last.output) > 16 else ""))
    if rates:
        mean, spread = sum(rates) / len(rates), (max(rates) - min(rates)) / 2
        print(f"Pipeline Generation Speed: {mean:.2f} +- {spread:.2f} tok/s ({len(rates)} runs)")
    return 0


def _teacher_force(args, eng, ids, n_predict, chunk) -> int:
    """Feeds prompt ++ reference ids and compares every step's top-1 with the reference; with
    --dump-logits writes "CLBRLGT1", u32 n, u32 vocab, n x vocab float32 (src/main.c:1333-1351).
    The row after stream position q predicts reference step q - (n_prompt - 1) (:1379-1384).
    Without --teacher-force the model's own greedy tokens are fed and dumped."""
    import torch
    from .csrc import ops
    from .engine.batch import StepEntry
    V = eng.model.vocab_size
    ref = _ids_from(args.teacher_force)[:n_predict] if args.teacher_force else None
    n = len(ref) if ref is not None else n_predict
    fout = None
    if args.dump_logits:
        fout = open(args.dump_logits, "wb")
        fout.write(b"CLBRLGT1" + struct.pack("<II", 0, V))
    eng.begin("tf")
    # the prompt, all but its last token, in portions
    for i in range(0, len(ids) - 1, chunk):
        eng.step([StepEntry("tf", ids[i:min(i + chunk, len(ids) - 1)], [])])
    rows_written = agree = 0
    pending = [ids[-1]]
    step = 0
    mismatches = []
    while step < n:
        if ref is not None:
            take = min(max(1, args.tf_batch), n - step)
            feed = pending + ref[step:step + take - 1]
        else:
            take, feed = 1, pending
        logits = eng.step([StepEntry("tf", feed, list(range(len(feed))))])
        picked = torch.empty(len(feed), dtype=torch.int32, device=logits.device)
        ops.argmax(logits, picked)                         # ties go to the lowest id, as in generation
        top = picked.cpu().tolist()
        if fout is not None:
            logits.cpu().numpy().astype("<f4").tofile(fout)
            rows_written += len(feed)
        if ref is not None:
            for j in range(take):
                if top[j] == ref[step + j]:
                    agree += 1
                else:
                    mismatches.append((step + j, top[j], ref[step + j]))
            pending = [ref[step + take - 1]]
        else:
            print(top[0])
            pending = [top[0]]
        step += take
    eng.end("tf")
    if fout is not None:
        fout.seek(8)
        fout.write(struct.pack("<I", rows_written))
        fout.close()
    if ref is not None:
        print(f"teacher-force: top-1 agreement {agree}/{n}", file=sys.stderr)
        for s, got, want in mismatches[:8]:
            print(f"  step {s}: model {got}, reference {want}", file=sys.stderr)
        return 0 if agree == n else 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
