"""Compiles the HIP sources of this folder for gfx950 with hipcc, one shared library a source,
and the plain C interface (capi.cpp, host code only) with the C++ compiler against libpython.

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

# Host-only libraries: name -> (source, further files whose change makes it stale)
HOST_MODULES = {
    "amd": ("capi.cpp", ["../../include/tuff_amd.h"]),     # libtuff_amd.so, the plain C interface
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


def _host_command() -> list[str]:
    """Compiler and flags for a host-only library that embeds the Python interpreter."""
    import sysconfig
    cxx = next((c for c in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"),
                            shutil.which("clang++"), "/opt/rocm/llvm/bin/clang++") if c and shutil.which(c)), None)
    if cxx is None:
        raise BuildError("no C++ compiler found (looked at $CXX, g++, c++, clang++)")
    v = sysconfig.get_config_vars()
    libdirs = [d for d in (v.get("LIBPL"), v.get("LIBDIR")) if d]
    return ([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall",
             "-I", sysconfig.get_paths()["include"]]
            + [f"-L{d}" for d in libdirs] + [f"-Wl,-rpath,{d}" for d in libdirs[1:]]
            + [f"-lpython{v['LDVERSION']}", "-ldl", "-lpthread"])


def _source_hash(module: str) -> str:
    h = hashlib.sha256()
    if module in HOST_MODULES:
        src, more = HOST_MODULES[module]
        files, flags = [src] + more, _host_command()
    else:
        files, flags = [MODULES[module]] + HEADERS, FLAGS
    for fn in files:
        with open(os.path.join(HERE, fn), "rb") as f:
            h.update(f.read())
    h.update(" ".join(flags).encode())
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
    if module not in MODULES and module not in HOST_MODULES:
        raise BuildError(f"unknown module '{module}'; known: {sorted(MODULES) + sorted(HOST_MODULES)}")
    host = module in HOST_MODULES
    name = HOST_MODULES[module][0] if host else MODULES[module]
    src = os.path.join(HERE, name)
    out_dir = _writable_dir()
    out = os.path.join(out_dir, f"libtuff_{module}.so")
    tmp = os.path.join(out_dir, f".libtuff_{module}.{os.getpid()}.{threading.get_ident()}.so")
    if host:
        cmd = _host_command()
        cmd = cmd[:1] + [src, "-o", tmp] + cmd[1:]          # libraries after the source that needs them
    else:
        cmd = [_hipcc()] + FLAGS + ["-I", HERE, "-o", tmp, src]
    if not quiet:
        _say(f"compiling {name}" + ("" if host else f" for {ARCH}") + " ...")
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)            # hipcc wants somewhere to keep temporaries
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    done = threading.Event()

    def ticker():
        while not done.wait(10.0):
            if not quiet:
                _say(f"  still compiling {name} ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    log, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise BuildError(f"{os.path.basename(cmd[0])} failed on {name} (exit {proc.returncode}):\n{log}")
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
    every = list(MODULES) + list(HOST_MODULES)
    todo = [m for m in every if force or find_built(m) is None]
    out = {m: find_built(m) for m in every if m not in todo}
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo) or 1))) as ex:
        for m, path in zip(todo, ex.map(compile_module, todo)):
            out[m] = path
    return out


if __name__ == "__main__":
    build_all(force="--stale-only" not in sys.argv)
