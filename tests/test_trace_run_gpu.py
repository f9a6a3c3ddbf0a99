"""bin/trace_run as a user runs it: a subprocess fed JSON lines, logits files
read back and compared with the plain implementation, in both dtypes, with the
pool sized by --max-tokens so that pages are used again."""
import os
import subprocess
import sys

import numpy as np
import pytest

import traces
from helpers import CONFIGS, random_tokens, read_folder
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

LENGTHS = {"a": 97, "b": 45, "c": 70, "d": 33, "e": 51}
PROMPTS = {"a": 60, "b": 12, "c": 41, "d": 30, "e": 2}
ROUNDED = plain.bf16_sites(("gemm_in", "kv_cache", "q"))


def run_trace(folder, dtype, trace, out_dir, options=None):
    n_tok = traces.max_tokens(trace)
    proc = subprocess.Popen([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                             "--out", out_dir] + (options if options is not None else ["--max-tokens", str(n_tok)]),
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    # one step at a time: the next one only after `done <step>`
    for i, line in enumerate(traces.to_jsonl(trace).splitlines()):
        proc.stdin.write(line + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {i}"
    proc.stdin.close()
    assert proc.wait(timeout=120) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_trace_run_mixed(model_folders, tmp_path, name, dtype):
    folder = model_folders(name, "bfloat16", True)
    cfg, w = read_folder(folder)
    V = cfg["vocab_size"]
    requests = {r: random_tokens(n, V, 90 + i) for i, (r, n) in enumerate(LENGTHS.items())}
    trace = traces.mixed(requests, PROMPTS, live=4)
    out = str(tmp_path / "out")
    run_trace(folder, dtype, trace, out)
    exact = {r: plain.forward(w, cfg, t) for r, t in requests.items()}
    if dtype == "float32":
        want, tol = exact, 2e-5
    else:
        want = {r: plain.forward(w, cfg, t, ROUNDED) for r, t in requests.items()}
        tol = 1.0 * max(np.abs(want[r] - exact[r]).max() for r in want)
    fed = {r: 0 for r in requests}
    worst = 0.0
    for i, step in enumerate(trace):
        n_want = sum(len(wn) for _, _, wn in step["entries"])
        rows = np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(n_want, V)
        k = 0
        for r, toks, wn in step["entries"]:
            for j in wn:
                worst = max(worst, float(np.abs(rows[k] - want[r][fed[r] + j]).max()))
                k += 1
            fed[r] += len(toks)
    print(f"\n[trace_run {name} {dtype}] max |engine - plain| = {worst:.3e} (allowed {tol:.3e})")
    assert worst < tol


def test_trace_run_writes_only_what_is_wanted(model_folders, tmp_path):
    folder = model_folders("A")
    trace = [{"entries": [("r", [1, 2, 3, 4], [])], "end": []},
             {"entries": [("r", [5, 6], [1]), ("s", [9, 8, 7], [0, 2])], "end": ["s"]},
             {"entries": [("r", [7], [0])], "end": ["r"]}]
    out = str(tmp_path / "out")
    run_trace(folder, "float32", trace, out)
    assert sorted(os.listdir(out)) == ["1.f32", "2.f32", "index.jsonl"]
    import json
    index = [json.loads(line) for line in open(os.path.join(out, "index.jsonl"))]
    assert index == [{"step": 1, "request": "r", "position": 5, "file": "1.f32", "row": 0},
                     {"step": 1, "request": "s", "position": 0, "file": "1.f32", "row": 1},
                     {"step": 1, "request": "s", "position": 2, "file": "1.f32", "row": 2},
                     {"step": 2, "request": "r", "position": 6, "file": "2.f32", "row": 0}]
    assert os.path.getsize(os.path.join(out, "1.f32")) == 3 * 256 * 4
    cfg, w = read_folder(folder)
    rows = np.fromfile(os.path.join(out, "1.f32"), dtype="<f4").reshape(3, 256)
    assert np.abs(rows[0] - plain.forward(w, cfg, [1, 2, 3, 4, 5, 6])[5]).max() < 2e-5
    assert np.abs(rows[2] - plain.forward(w, cfg, [9, 8, 7])[2]).max() < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_from_a_configuration_alone(tmp_path, dtype):
    """`--random-weights --seed` from a folder that holds config.json and nothing else, the pool given in pages
    (as few as the trace needs), more live requests than the default allows: the logits are the plain model's
    on the weights that `write_model_folder` writes for the same configuration and seed, and index.jsonl
    names the file and row of every (step, request, position)."""
    import json
    from tinyinfer_amd.weights import write_model_folder
    cfg = CONFIGS["B"]
    bare = tmp_path / "bare"
    bare.mkdir()
    (bare / "config.json").write_text(json.dumps(cfg))
    full = str(tmp_path / "full")
    write_model_folder(full, cfg, seed=77, dtype=dtype)       # (a 32-bit engine draws 32-bit matrices: nothing is rounded)
    _, w = read_folder(full)
    V = cfg["vocab_size"]
    requests = {f"r{i}": random_tokens(20 + 3 * i, V, 40 + i) for i in range(10)}
    trace = traces.mixed(requests, {r: 5 + i for i, r in enumerate(requests)}, live=10)
    assert max(len(s["entries"]) for s in trace) > 8
    out = str(tmp_path / "deep" / "out")
    pages = traces.max_pages(trace, 4)
    run_trace(str(bare), dtype, trace, out, ["--random-weights", "--seed", "77", "--num-pages", str(pages), "--page-size", "4",
                                             "--max-requests", "10", "--max-seq", "64"])
    exact = {r: plain.forward(w, cfg, t) for r, t in requests.items()}
    if dtype == "float32":
        want, tol = exact, 2e-5
    else:
        want = {r: plain.forward(w, cfg, t, ROUNDED) for r, t in requests.items()}
        tol = 1.0 * max(np.abs(want[r] - exact[r]).max() for r in want)
    index = [json.loads(line) for line in open(os.path.join(out, "index.jsonl"))]
    assert len(index) == sum(len(t) for t in requests.values())          # every token's logits were wanted
    assert {(e["request"], e["position"]) for e in index} == {(r, p) for r, t in requests.items() for p in range(len(t))}
    files = {}
    worst = 0.0
    for e in index:
        if e["file"] not in files:
            files[e["file"]] = np.fromfile(os.path.join(out, e["file"]), dtype="<f4").reshape(-1, V)
            assert e["file"] == f"{e['step']}.f32"
        worst = max(worst, float(np.abs(files[e["file"]][e["row"]] - want[e["request"]][e["position"]]).max()))
    print(f"\n[trace_run --random-weights {dtype}] max |engine - plain| = {worst:.3e} (allowed {tol:.3e})")
    assert worst < tol


def test_trace_run_refuses_what_it_cannot_serve(tmp_path):
    exe = os.path.join(ROOT, "bin", "trace_run")
    bad = subprocess.run([exe, "--model", str(tmp_path), "--dtype", "float32", "--out", str(tmp_path / "o")], capture_output=True,
                         text=True, stdin=subprocess.DEVNULL)
    assert bad.returncode == 2 and "--max-tokens or --num-pages" in bad.stderr
    missing = subprocess.run([exe, "--model", str(tmp_path / "nothing"), "--dtype", "float32", "--out", str(tmp_path / "o"),
                              "--max-tokens", "64"], capture_output=True, text=True, stdin=subprocess.DEVNULL)
    assert missing.returncode == 1 and "config.json" in missing.stderr
