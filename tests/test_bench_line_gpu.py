"""bench.py as the driver runs it: one JSON line with the contract's keys, at one layer of the default
sizes so that it takes seconds; greedy and with drawn tokens; and the refusal of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          cwd=ROOT, timeout=600)


def test_more_than_one_gpu_is_refused_in_one_line():
    """N > 1: one line that says so, exit code 2 (nothing of the GPU is touched before)."""
    done = run_bench("--gpus", "2", "--steps", "4", "--warmup", "1")
    assert done.returncode == 2
    lines = [l for l in done.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


@pytest.mark.gpu
@pytest.mark.parametrize("drawn", [False, True])
def test_bench_line_keeps_the_contract(drawn):
    args = ["--layers", "1", "--steps", "6", "--warmup", "2", "--no-peaks"]
    if drawn:
        args += ["--temperature", "0.8", "--top-p", "0.95"]
    done = run_bench(*args)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [l for l in done.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 6 and out["warmup"] == 2 and out["higher_is_better"] is True
    assert out["unit"] == "tokens/s" and out["dtype"] == "bf16" and "synthetic" in out["data"]
    assert out["value"] > 0 and out["ms_per_step"] > 0
    assert abs(out["value"] - out["config"]["global_batch"] / (out["ms_per_step"] * 1e-3)) < 0.01 * out["value"]
    cfg = out["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())      # flat, at most 20 keys
    assert cfg["layers"] == 1 and cfg["layers_in_config"] == 28                               # both numbers are named
    assert cfg["hidden"] == 1024 and cfg["vocab"] == 151936 and cfg["global_batch"] == 8 and cfg["cached_tokens"] == 2048
    assert cfg["sampling"] == ("temperature 0.8 top-k 512 top-p 0.95" if drawn else "greedy")
    assert set(out["prefill"]) >= {"value", "tokens", "ms", "frac"} and out["prefill"]["tokens"] == 2048
    assert set(out["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac"}
    assert out["roofline"]["bound"] == "hbm" and out["roofline"]["peak"] == 8000.0 and out["roofline"]["unit"] == "GB/s"
    assert abs(out["roofline"]["frac"] - out["roofline"]["achieved"] / out["roofline"]["peak"]) < 1e-3
    assert set(out["points"]) == {"decode_b1", "decode_b64"} and all(v > 0 for v in out["points"].values())
    # the figures behind the fractions, worked out here by hand for this configuration (one layer): every matrix of
    # the layer and the tied head once, norm vectors in 32-bit, keys and values of 8 requests at their mean length
    layer, head = (4096 + 2048 + 3 * 3072) * 1024, 151936 * 1024
    weight_bytes = (layer + head) * 2 + (2 * 1024 + 2 * 128 + 1024) * 4
    kv_bytes = 8 * (2048 + 2 + 6 / 2) * 2 * 8 * 128 * 2
    achieved = (weight_bytes + kv_bytes) / (out["ms_per_step"] * 1e-3) / 1e9
    assert abs(out["roofline"]["achieved"] - achieved) < 0.01 * achieved, (out["roofline"]["achieved"], achieved)
    flops = 2.0 * layer * 2048 + 2.0 * head + 2.0 * 128 * 2048 * 2049 * 16
    frac = flops / (out["prefill"]["ms"] * 1e-3) / 2.5e15
    assert abs(out["prefill"]["frac"] - frac) < 0.01 * frac + 1e-4, (out["prefill"]["frac"], frac)
    assert abs(out["prefill"]["value"] - 2048 / (out["prefill"]["ms"] * 1e-3)) < 0.01 * out["prefill"]["value"]
