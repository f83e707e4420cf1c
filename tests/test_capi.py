"""The plain C interface (include/tuff_amd.h): a C program, compiled here, drives the library as
a child process.  Without a GPU: writing a random model folder and the sampling defaults.  On
the GPU: the step function, generation and the scheduler calls against the Python entry point
and the plain implementation."""
import filecmp
import json
import os
import shutil
import subprocess

import numpy as np
import pytest
import torch

import util

CC = shutil.which("gcc") or shutil.which("cc") or shutil.which("clang")


@pytest.fixture(scope="module")
def client(tmp_path_factory):
    """Path of the compiled tests/capi_client.c, linked against the built library."""
    from tuff_amd.csrc import build
    if CC is None:
        pytest.skip("no C compiler")
    lib = build.ensure_built("amd")
    libdir = os.path.dirname(lib)
    exe = str(tmp_path_factory.mktemp("capi") / "capi_client")
    subprocess.run([CC, "-std=c11", "-D_GNU_SOURCE", "-Wall", "-Werror", os.path.join(util.ROOT, "tests", "capi_client.c"),
                    "-I", os.path.join(util.ROOT, "include"), f"-L{libdir}", "-ltuff_amd",
                    f"-Wl,-rpath,{libdir}", "-o", exe], check=True)
    return exe


def run_client(exe, *args, timeout=600):
    env = dict(os.environ)
    env.pop("PYTHONPATH", None)                      # the library finds the package by itself
    return subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=timeout,
                          env=env, cwd="/")


def test_write_random_model_and_defaults_from_c(client, tmp_path):
    from tuff_amd.models.registry import config_from_dict
    from tuff_amd.sampling.params import SamplingParams
    from tuff_amd.weights.random_init import write_random_model
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(util.TINY_B))
    p = run_client(client, "write-random", cfg_file, 5, tmp_path / "from_c", "bfloat16")
    assert p.returncode == 0, p.stderr
    write_random_model(config_from_dict(util.TINY_B), str(tmp_path / "from_py"), 5, torch.bfloat16)
    for name in ("config.json", "model.safetensors"):
        assert filecmp.cmp(tmp_path / "from_c" / name, tmp_path / "from_py" / name, shallow=False), name
    d = SamplingParams()
    want = f"defaults {d.temp:g} {d.top_p:g} {d.top_k} {d.min_p:g} {d.repeat_penalty:g} {d.repeat_last_n} " \
           f"{d.seed} {d.max_new_tokens} {int(d.ignore_eos)}"
    assert want in p.stdout


def test_failure_gives_a_code_and_a_message(client, tmp_path):
    p = run_client(client, "write-random", tmp_path / "missing.json", 5, tmp_path / "out", "bfloat16")
    assert p.returncode == 1
    assert "FileNotFoundError" in p.stderr and "missing.json" in p.stderr
    bad = tmp_path / "bad.json"
    bad.write_text(json.dumps({"architectures": ["NoSuchModel"]}))
    p = run_client(client, "write-random", bad, 5, tmp_path / "out", "bfloat16")
    assert p.returncode == 1 and "NoSuchModel" in p.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_c_program_steps_generates_and_schedules(gpu, client, tmp_path, dtype):
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    name = "B"
    stored = "float32" if dtype == "float32" else "bfloat16"
    folder = util.model_folder(name, stored)
    V = util.TINY_B["vocab_size"]
    prompt = util.rand_tokens(41, V, 12)
    n_new = 9
    logits_file = tmp_path / "logits.f32"
    p = run_client(client, "run", folder, dtype, logits_file, n_new, ",".join(map(str, prompt)))
    assert p.returncode == 0, p.stdout + p.stderr
    lines = dict(l.split(" ", 1) if " " in l else (l, "") for l in p.stdout.splitlines())
    assert lines["vocab"].split()[0] == str(V)
    assert lines["length"] == f"{len(prompt)} 5"
    assert lines["length-after-errors"] == str(len(prompt))
    assert "99" in lines["error-unknown:"] and "room" in lines["error-room:"]
    assert "closed" in lines

    # the step function's logits at every position against the plain implementation
    got = torch.from_numpy(np.fromfile(logits_file, dtype="<f4").reshape(len(prompt), V).copy())
    util.assert_close(dtype, got, util.expected(name, prompt, stored), "C step")

    # generation and the scheduler calls against the Python entry point in this process
    llm = LLM(folder, dtype=dtype, max_num_seqs=4, ctx_size=512)
    base = SamplingParams(max_new_tokens=n_new, ignore_eos=True)
    here = llm.generate([prompt], base)[0]
    assert lines["generate"].split() == [str(t) for t in here.token_ids]

    def sched_line(r):
        key = next(k for k in p.stdout.splitlines() if k.startswith(f"sched {r} "))
        head, toks = key.split(":")
        return int(head.split()[-1]), [int(t) for t in toks.split()]
    warm = SamplingParams(temp=0.8, top_k=20, top_p=0.9, seed=11, max_new_tokens=n_new + 3, ignore_eos=True)
    short = SamplingParams(max_new_tokens=3, ignore_eos=True)
    alone = [llm.generate([pr], sp)[0].token_ids
             for pr, sp in ((prompt, base), (prompt[2:], warm), (prompt[1:], short))]
    for r in range(3):
        fin, toks = sched_line(r)
        assert fin == 2                                             # TUFF_FINISH_LENGTH
        assert len(toks) == len(alone[r])
        if dtype == "float32":
            assert toks == alone[r], f"request {r}: batched through C differs from alone in Python"
    assert sched_line(0)[1] == here.token_ids or dtype == "bfloat16"
    assert lines["rejected:"] == "left 0 events 1 request 5 token -1 finished 6"
