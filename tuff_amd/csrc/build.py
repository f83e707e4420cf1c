"""Compiles the HIP sources of this folder for gfx950 with hipcc, one shared library a source.

A library is rebuilt when the hash of its source, the shared header and the flags differs
from the one recorded beside it; otherwise the built file is loaded as it is.  Libraries go
to `_lib/` beside the sources, or, where that folder cannot be written, to
`$TUFF_AMD_BUILD_DIR` or a per-user folder under the system's temporary directory.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
# -packed-fp32-ops off: the compiler must not form packed float32 instructions.
FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-shared", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
         # MFMA results in ordinary vector registers: without this the compiler parks accumulators in
         # the accumulation registers and copies them back and forth around every non-matrix use
         "-mllvm", "-amdgpu-mfma-vgpr-form=1"]
HEADERS = ["common.h"]

MODULES = {
    "elementwise": "elementwise.hip",
    "gemm_f32": "gemm_f32.hip",
    "gemm_bf16": "gemm_bf16.hip",
    "rope_kv": "rope_kv.hip",
    "attention": "attention.hip",
    "attention_mfma": "attention_mfma.hip",
    "attention_prefill": "attention_prefill.hip",
    "shortconv": "shortconv.hip",
    "sampling": "sampling.hip",
}


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels "
                     "cannot be compiled and there is no fallback path")


def _writable_dir() -> str:
    cands = [os.environ.get("TUFF_AMD_BUILD_DIR"), os.path.join(HERE, "_lib"),
             os.path.join(tempfile.gettempdir(), f"tuff_amd_lib_{os.getuid()}")]
    for d in cands:
        if not d:
            continue
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}_{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.unlink(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the compiled kernels; set TUFF_AMD_BUILD_DIR")


def _source_hash(module: str) -> str:
    h = hashlib.sha256()
    for fn in [MODULES[module]] + HEADERS:
        with open(os.path.join(HERE, fn), "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()


def _candidates(module: str):
    dirs = [os.environ.get("TUFF_AMD_BUILD_DIR"), os.path.join(HERE, "_lib"),
            os.path.join(tempfile.gettempdir(), f"tuff_amd_lib_{os.getuid()}")]
    for d in dirs:
        if d:
            yield os.path.join(d, f"libtuff_{module}.so")


def find_built(module: str) -> str | None:
    """Path of an up-to-date built library of `module`, or None."""
    want = _source_hash(module)
    for path in _candidates(module):
        try:
            with open(path + ".hash") as f:
                if f.read().strip() == want and os.path.isfile(path):
                    return path
        except OSError:
            continue
    return None


def _say(msg: str) -> None:
    print(f"[tuff_amd] {msg}", file=sys.stderr, flush=True)


def compile_module(module: str, quiet: bool = False) -> str:
    """Compiles one module unconditionally and returns the path of the library."""
    if module not in MODULES:
        raise BuildError(f"unknown kernel module '{module}'; known: {sorted(MODULES)}")
    src = os.path.join(HERE, MODULES[module])
    out_dir = _writable_dir()
    out = os.path.join(out_dir, f"libtuff_{module}.so")
    tmp = os.path.join(out_dir, f".libtuff_{module}.{os.getpid()}.{threading.get_ident()}.so")
    cmd = [_hipcc()] + FLAGS + ["-I", HERE, "-o", tmp, src]
    if not quiet:
        _say(f"compiling {MODULES[module]} for {ARCH} ...")
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)            # hipcc wants somewhere to keep temporaries
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    done = threading.Event()

    def ticker():
        while not done.wait(10.0):
            if not quiet:
                _say(f"  still compiling {MODULES[module]} ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    log, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise BuildError(f"hipcc failed on {MODULES[module]} (exit {proc.returncode}):\n{log}")
    os.replace(tmp, out)
    with open(out + ".hash.tmp", "w") as f:
        f.write(_source_hash(module))
    os.replace(out + ".hash.tmp", out + ".hash")
    if not quiet:
        _say(f"  built {os.path.basename(out)} in {time.time() - t0:.1f} s")
    return out


def ensure_built(module: str) -> str:
    """Path of the library of `module`; compiles it first if no current build exists."""
    path = find_built(module)
    if path is None:
        path = compile_module(module)
    return path


def build_all(force: bool = True, jobs: int = 8) -> dict[str, str]:
    """Compiles every module (in parallel).  With force=False only the missing or stale ones."""
    from concurrent.futures import ThreadPoolExecutor
    todo = [m for m in MODULES if force or find_built(m) is None]
    out = {m: find_built(m) for m in MODULES if m not in todo}
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo) or 1))) as ex:
        for m, path in zip(todo, ex.map(compile_module, todo)):
            out[m] = path
    return out


if __name__ == "__main__":
    build_all(force="--stale-only" not in sys.argv)
