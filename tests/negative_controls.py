"""Negative controls: one realistic bug at a time is put into a scratch copy of the package, and the
tests named for it must go red there.  A test suite that stays green under a mutant has a blind spot.

The table (negative_controls.txt beside this file) holds, per control: an id, the file, the exact text
to replace (it must occur exactly once: a control whose text has moved on is stale, which is an error),
its replacement, and the checks (pytest node ids) that must fail.  The scratch copy holds the package,
the tests and the programs; kernels of a mutated source are compiled into a folder of the control's own
(`_negctl/<id>/` beside this file, or a temporary folder), everything unmutated is loaded from where the
real tree keeps it.  Every mutant reads only memory that the unmutated code may read, so none can fault.

The idea and the first controls (conv taps swapped, gate from the wrong third, attention that sees the
next token of its batch, a portion's positions off by one) follow the reference's
tests/lfm25_negative_controls.sh and tests/lfm25_negctl.txt:1-23, :33-40, :108-114, :148-154.

    python tests/negative_controls.py --list
    python tests/negative_controls.py --build        compile every mutant's kernels now (no GPU needed)
    python tests/negative_controls.py [--only ID]    run on a GPU: baseline first, then every mutant
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
TABLE = os.path.join(HERE, "negative_controls.txt")
COPIED = ("tuff_amd", "tests", "bin", "include", "bench.py", "__graft_entry__.py")
SKIPPED_DIRS = {"__pycache__", "_lib", "_negctl", ".pytest_cache"}


class StaleControl(RuntimeError):
    pass


def _unescape(s: str) -> str:
    out, i = [], 0
    while i < len(s):
        if s[i] == "\\" and i + 1 < len(s) and s[i + 1] in "n\\":
            out.append("\n" if s[i + 1] == "n" else "\\")
            i += 2
        else:
            out.append(s[i])
            i += 1
    return "".join(out)


def read_table(path: str = TABLE) -> list[dict]:
    """Records separated by blank lines, `key: value` a line, '#' comments; in `old` and `new` "\\n" is a
    newline and "\\\\" a backslash, and everything after the one space behind the colon counts."""
    controls, cur = [], {}
    with open(path) as f:
        for raw in f:
            line = raw.rstrip("\n")
            if not line.strip():
                if cur:
                    controls.append(cur)
                    cur = {}
                continue
            if line.lstrip().startswith("#"):
                continue
            key, sep, value = line.partition(":")
            if not sep:
                raise ValueError(f"{path}: not a 'key: value' line: {line!r}")
            cur[key.strip()] = value[1:] if value.startswith(" ") else value
    if cur:
        controls.append(cur)
    for c in controls:
        missing = [k for k in ("id", "desc", "file", "old", "new", "checks") if k not in c]
        if missing:
            raise ValueError(f"{path}: control {c.get('id', '?')!r} lacks {missing}")
        c["old"], c["new"] = _unescape(c["old"]), _unescape(c["new"])
        c["checks"] = c["checks"].split()
    ids = [c["id"] for c in controls]
    if len(set(ids)) != len(ids):
        raise ValueError(f"{path}: an id appears twice")
    return controls


def make_scratch(dst: str) -> str:
    """A copy of the tree's sources under dst (no built files, no caches).  Returns dst."""
    for name in COPIED:
        src = os.path.join(ROOT, name)
        if os.path.isdir(src):
            shutil.copytree(src, os.path.join(dst, name), symlinks=True,
                            ignore=lambda d, names: [n for n in names if n in SKIPPED_DIRS or n.endswith((".pyc", ".so"))])
        elif os.path.isfile(src):
            shutil.copy2(src, os.path.join(dst, name))
    # kernels of unmutated sources are found where the real tree has them (same hash), never compiled again
    real_lib = os.path.join(ROOT, "tuff_amd", "csrc", "_lib")
    if os.path.isdir(real_lib):
        os.symlink(real_lib, os.path.join(dst, "tuff_amd", "csrc", "_lib"))
    return dst


def apply(control: dict, scratch: str) -> str:
    """Puts the control's bug into the scratch copy.  Returns the path of the changed file."""
    path = os.path.join(scratch, control["file"])
    with open(path) as f:
        text = f.read()
    n = text.count(control["old"])
    if n != 1:
        raise StaleControl(f"control {control['id']}: its text occurs {n} times in {control['file']}, not once; "
                           f"the source has moved on, bring the table up to date")
    with open(path, "w") as f:
        f.write(text.replace(control["old"], control["new"]))
    return path


def revert(control: dict, scratch: str) -> None:
    shutil.copy2(os.path.join(ROOT, control["file"]), os.path.join(scratch, control["file"]))


def build_dir(control: dict) -> str:
    """Where the mutant's kernels are built: beside this file if that can be written, else a temporary folder."""
    for base in (os.path.join(HERE, "_negctl"), os.path.join(tempfile.gettempdir(), f"tuff_amd_negctl_{os.getuid()}")):
        d = os.path.join(base, control["id"])
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}")
            open(probe, "w").close()
            os.unlink(probe)
            return d
        except OSError:
            continue
    raise RuntimeError("no folder to build the mutants' kernels in")


def _env(scratch: str, control: dict | None) -> dict:
    env = dict(os.environ)
    env["PYTHONPATH"] = scratch
    env.pop("TUFF_AMD_BUILD_DIR", None)
    if control is not None:
        env["TUFF_AMD_BUILD_DIR"] = build_dir(control)
    return env


def module_of(control: dict) -> str | None:
    """The kernel module a control's file belongs to, or None for a Python file."""
    base = os.path.basename(control["file"])
    return base[:-4] if base.endswith(".hip") else None


def compile_mutant(control: dict, scratch: str) -> None:
    """Compiles the mutated kernel source of an applied control (a no-op if it is built already)."""
    mod = module_of(control)
    if mod is None:
        return
    code = f"from tuff_amd.csrc import build; build.ensure_built({mod!r})"
    p = subprocess.run([sys.executable, "-c", code], cwd=scratch, env=_env(scratch, control), capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError(f"control {control['id']}: the mutant does not compile:\n{p.stdout}\n{p.stderr}")


def run_checks(scratch: str, checks: list[str], control: dict | None, timeout: int = 600) -> dict:
    """Runs the checks with pytest in the scratch copy.  Returns {check: 'passed' | 'failed' | 'error' | 'missing'}."""
    cmd = [sys.executable, "-m", "pytest", "-q", "-rA", "-p", "no:cacheprovider", "--timeout", "120",
           "--timeout-method", "thread", *checks]
    p = subprocess.run(cmd, cwd=scratch, env=_env(scratch, control), capture_output=True, text=True, timeout=timeout)
    out = {c: "missing" for c in checks}
    for line in p.stdout.splitlines():
        word, _, rest = line.partition(" ")
        if word in ("PASSED", "FAILED", "ERROR"):
            node = rest.split(" - ")[0].strip()
            if node in out:
                out[node] = {"PASSED": "passed", "FAILED": "failed", "ERROR": "error"}[word]
    out["_log"] = p.stdout[-4000:] + p.stderr[-2000:]
    return out


def prebuild(quiet: bool = False, jobs: int = 6) -> None:
    """Compiles every mutant's kernels (on any machine with hipcc; no GPU needed), several at a time,
    each worker in a scratch copy of its own."""
    import threading
    from concurrent.futures import ThreadPoolExecutor
    todo = [c for c in read_table() if module_of(c) is not None]
    with tempfile.TemporaryDirectory(prefix="tuff_amd_negctl_") as tmp:
        local = threading.local()

        def build_one(c):
            if not hasattr(local, "tree"):
                local.tree = make_scratch(os.path.join(tmp, f"tree_{threading.get_ident()}"))
            apply(c, local.tree)
            try:
                compile_mutant(c, local.tree)
            finally:
                revert(c, local.tree)
            if not quiet:
                print(f"[negative controls] {c['id']}: built", file=sys.stderr, flush=True)

        with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as ex:
            list(ex.map(build_one, todo))


def main(argv) -> int:
    controls = read_table()
    if "--list" in argv:
        for c in controls:
            print(f"{c['id']:40s} {c['file']:40s} {c['desc']}")
        return 0
    if "--build" in argv:
        prebuild()
        return 0
    only = argv[argv.index("--only") + 1] if "--only" in argv else None
    chosen = [c for c in controls if only in (None, c["id"])]
    if not chosen:
        print(f"no control {only!r}", file=sys.stderr)
        return 2
    bad = 0
    with tempfile.TemporaryDirectory(prefix="tuff_amd_negctl_") as tmp:
        scratch = make_scratch(os.path.join(tmp, "tree"))
        every = sorted({k for c in chosen for k in c["checks"]})
        base = run_checks(scratch, every, None)
        broken = [k for k in every if base[k] != "passed"]
        if broken:
            print(f"the unmutated tree does not pass {broken}:\n{base['_log']}", file=sys.stderr)
            return 1
        print(f"baseline: {len(every)} checks pass")
        for c in chosen:
            apply(c, scratch)
            try:
                compile_mutant(c, scratch)
                res = run_checks(scratch, c["checks"], c)
            finally:
                revert(c, scratch)
            verdict = "CAUGHT" if all(res[k] == "failed" for k in c["checks"]) else "NOT CAUGHT"
            bad += verdict != "CAUGHT"
            print(f"{c['id']:40s} {verdict}  " + " ".join(f"{k.split('::')[-1]}={res[k]}" for k in c["checks"]))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
