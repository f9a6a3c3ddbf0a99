"""A part kind, its kernels and an architecture added from outside the framework, in C++: the test
builds a kernel library (tests/cpp/toy_relu.hip) and a plugin (tests/cpp/plugin_part.cpp, against
include/inference.h), and the model made of them is written, loaded, replayed through bin/trace_run
and stepped through the Python entry point without a change to a file under the framework's folder.
(The reference's one architecture is a string compare in its loader, /root/reference/src/model.cpp:26-30.)"""
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

import traces
from helpers import random_tokens, read_folder
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")

CFG = dict(architectures=["ToyCppLM"], vocab=131, hidden=48, heads=3, kv_heads=1, head_dim=16, inner=72, alpha=0.7, layers=2,
           eps=1e-5, theta=1e4)


@pytest.fixture(scope="module")
def plugin(tmp_path_factory):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.csrc import build
    d = tmp_path_factory.mktemp("plugin")
    kernels = str(d / "libtoy_relu.so")
    done = subprocess.run([build._hipcc(), "-O2", "--offload-arch=gfx950", "-fPIC", "-shared", os.path.join(CPP, "toy_relu.hip"),
                           "-o", kernels], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    host = build.ensure_host()
    lib = str(d / "libtoy_plugin.so")
    cxx = shutil.which("g++") or shutil.which("c++")
    done = subprocess.run([cxx, "-std=c++17", "-O1", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(build.PKG, "include"),
                           "-I" + os.path.join(build.ROCM, "include"), os.path.join(CPP, "plugin_part.cpp"), "-o", lib, host,
                           "-Wl,-rpath," + os.path.dirname(host)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    os.environ["TOY_RELU_LIB"] = kernels
    return lib


def toy_forward(w, toks, rnd):
    c = CFG
    T = len(toks)
    x = plain.embed(w["emb.weight"], toks)
    for i in range(c["layers"]):
        p = f"l.{i}"
        h = rnd("gemm_in", plain.rms_norm(x, w[p + ".n1.weight"], c["eps"]))
        a = p + ".attn"
        q = plain.linear(h, w[a + ".q_proj.weight"]).reshape(T, c["heads"], c["head_dim"])
        k = plain.linear(h, w[a + ".k_proj.weight"]).reshape(T, c["kv_heads"], c["head_dim"])
        v = plain.linear(h, w[a + ".v_proj.weight"]).reshape(T, c["kv_heads"], c["head_dim"])
        q = plain.qk_norm(q, w[a + ".q_norm.weight"], c["eps"])
        k = plain.qk_norm(k, w[a + ".k_norm.weight"], c["eps"])
        q = rnd("q", plain.rope_neox(q, range(T), c["theta"]))
        k = rnd("kv_cache", plain.rope_neox(k, range(T), c["theta"]))
        o = plain.attention(q, k, rnd("kv_cache", v), None).reshape(T, -1)
        x = x + plain.linear(rnd("gemm_in", o), w[a + ".o_proj.weight"])
        h = rnd("gemm_in", plain.rms_norm(x, w[p + ".n2.weight"], c["eps"]))
        y = rnd("gemm_in", c["alpha"] * np.maximum(plain.linear(h, w[p + ".ffn.w1"]), 0.0))
        x = x + plain.linear(y, w[p + ".ffn.w2"])
    return plain.linear(rnd("gemm_in", plain.rms_norm(x, w["norm.weight"], c["eps"])), w["emb.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_part_and_an_architecture_from_a_plugin(plugin, tmp_path, dtype):
    import tinyinfer_amd as ti
    ti.load_plugin(plugin)
    assert "toy_relu" in ti.parts.registered_parts("ffn") and "ToyCppLM" in ti.registered_architectures()
    folder = str(tmp_path / "toy")
    ti.write_model_folder(folder, CFG, seed=3, dtype=dtype)
    _, w = read_folder(folder)
    assert w["l.1.ffn.w1"].shape == (72, 48) and abs(float(w["l.1.ffn.w1"].std()) - 0.2) < 0.02      # the part's own init
    requests = {r: random_tokens(n, CFG["vocab"], 20 + i) for i, (r, n) in enumerate({"a": 41, "b": 23, "c": 35}.items())}
    trace = traces.mixed(requests, {"a": 20, "b": 5, "c": 30}, live=2)
    out = str(tmp_path / "out")
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--plugin", plugin, "--model", folder, "--dtype", dtype, "--out", out,
                           "--num-pages", str(traces.max_pages(trace, 4)), "--page-size", "4", "--max-seq", "64"],
                          input=traces.to_jsonl(trace), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    assert proc.stdout.split() == [x for i in range(len(trace)) for x in ("done", str(i))]
    exact = {r: toy_forward(w, t, plain.no_rounding) for r, t in requests.items()}
    if dtype == "float32":
        want, tol = exact, 2e-5
    else:
        want = {r: toy_forward(w, t, plain.bf16_sites(("gemm_in", "kv_cache", "q"))) for r, t in requests.items()}
        tol = 1.0 * max(float(np.abs(want[r] - exact[r]).max()) for r in want)
    worst = 0.0
    files = {}
    for e in (json.loads(line) for line in open(os.path.join(out, "index.jsonl"))):
        if e["file"] not in files:
            files[e["file"]] = np.fromfile(os.path.join(out, e["file"]), dtype="<f4").reshape(-1, CFG["vocab"])
        worst = max(worst, float(np.abs(files[e["file"]][e["row"]] - want[e["request"]][e["position"]]).max()))
    print(f"\n[plugin part through trace_run, {dtype}] max |engine - plain| = {worst:.3e} (allowed {tol:.3e})")
    assert worst < tol
    # the same model through the Python entry point: the part shows as a view with its parameters and tensors
    engine = ti.Engine.from_folder(folder, dtype, page_size=4, max_tokens=128, max_requests=2, max_seq=64)
    ffn = engine.model.blocks[1].ffn
    assert (ffn.kind, ffn.inner, ffn.alpha) == ("toy_relu", 72, 0.7) and tuple(ffn.w2.shape) == (48, 72)
    logits = engine.step_graph([ti.StepEntry("a", requests["a"], [40])]).cpu().numpy()
    assert np.abs(logits[0] - want["a"][40]).max() < tol
    assert ti.generate_ids(engine, [requests["b"][:5]], max_new_tokens=4, use_graph=True)[0] == \
        ti.generate_ids(engine, [requests["b"][:5]], max_new_tokens=4)[0]
