"""The C++ programming interface: a program that includes inference.h alone (tests/cpp/api_program.cpp)
is built here, loads config B's folder, replays a mixed trace and runs a scheduled generation.  Its
float32 logits are those of the Python entry point bit for bit (both drive the same library), in
bfloat16 too, and its generated tokens are the same."""
import json
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest

import traces
from helpers import CONFIGS, random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def program(tmp_path_factory):
    """The program, compiled against the header and linked with the host library."""
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd import native
    from tinyinfer_amd.csrc import build
    native.ensure_kernels(["core", "gemm_generic", "attention_generic", "sampling", "gemm_bf16", "attention_bf16"])
    lib = build.ensure_host()
    out = str(tmp_path_factory.mktemp("cpp") / "api_program")
    cxx = shutil.which("g++") or shutil.which("c++")
    include = os.path.join(build.PKG, "include")
    cmd = [cxx, "-std=c++17", "-O1", "-I" + include, os.path.join(ROOT, "tests", "cpp", "api_program.cpp"), "-o", out,
           lib, "-Wl,-rpath," + os.path.dirname(lib), "-Wl,-rpath," + os.path.join(build.ROCM, "lib")]
    done = subprocess.run(cmd, capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    return out, os.path.dirname(lib)


def hip_runtime_env():
    """The program runs with the HIP runtime this process uses (torch brings its own)."""
    import torch
    env = dict(os.environ)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    env["LD_LIBRARY_PATH"] = torch_lib + os.pathsep + env.get("LD_LIBRARY_PATH", "")
    return env


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_program_equals_the_python_entry_point(program, model_folders, tmp_path, dtype):
    import tinyinfer_amd as ti
    exe, kernel_dir = program
    folder = model_folders("B", "bfloat16", True)
    V = CONFIGS["B"]["vocab_size"]
    requests = {"a": random_tokens(70, V, 1), "b": random_tokens(45, V, 2), "c": random_tokens(33, V, 3),
                "d": random_tokens(51, V, 4), "e": random_tokens(9, V, 5)}
    trace = traces.mixed(requests, {"a": 40, "b": 30, "c": 20, "d": 45, "e": 4})
    max_tokens = traces.max_tokens(trace)
    trace_file = tmp_path / "trace.jsonl"
    trace_file.write_text(traces.to_jsonl(trace))
    out = tmp_path / "out"
    out.mkdir()
    prompts = [random_tokens(n, V, 20 + n) for n in (5, 17, 33)]
    env = hip_runtime_env()
    env["TINYINFER_KERNEL_DIR"] = kernel_dir
    run = subprocess.run([exe, folder, dtype, str(trace_file), str(out), str(max_tokens), "4", json.dumps(prompts), "0.8",
                          "123", "7"], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0, run.stderr
    theirs = json.loads(run.stdout.strip().splitlines()[-1])

    engine = ti.Engine.from_folder(folder, dtype, page_size=4, max_tokens=max_tokens, max_requests=8, max_seq=max_tokens)
    n_files = 0
    for i, step in enumerate(trace):
        entries = [ti.StepEntry(r, toks, want) for r, toks, want in step["entries"]]
        logits = engine.step(entries) if entries else None
        for r in step["end"]:
            if engine.cache.has(r):
                engine.release(r)
        path = out / f"{i}.f32"
        if logits is None:
            assert not path.exists()
            continue
        mine = logits.cpu().numpy()
        got = np.fromfile(path, dtype="<f4").reshape(mine.shape)
        assert np.array_equal(got, mine), f"step {i}: the program's logits differ from the Python entry point's"
        n_files += 1
    assert n_files > 10
    want = ti.generate_ids(engine, prompts, max_new_tokens=6, temperature=0.8, seed=123, chunk_size=7, max_batched_tokens=16)
    assert theirs["generated"] == want
    assert theirs["steps"] > 6 and theirs["free_pages"] == engine.cache.num_free_pages()
