"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of Qwen3-0.6B with random weights in
bfloat16: a batch of 8 requests, each holding 2,048 cached tokens (filled by
real prefill steps), decoded for K steps through the serving path (scheduler's
step function from a captured graph, greedy sampling on the device, the sampled
token fed back).  One JSON line goes to stdout: `value` is decoded tokens a
second at batch 8; `points` has batch 1 and 64; `prefill` a 2,048-token prompt in
one step; `roofline` the decode step's bytes (every weight once, the cache of
the live requests) over its time against 8 TB/s.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

CONFIG = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=28, hidden_size=1024,
              num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072,
              vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              attention_bias=False, hidden_act="silu", max_position_embeddings=40960)
CONTEXT = 2048            # cached tokens each decoding request holds
MAX_SEQ = 4096            # context length a request may reach
PREFILL_TOKENS = 2048
PAGE = 16
PEAK_HBM = 8.0e12         # bytes/s, MI355X
PEAK_BF16 = 2.5e15        # dense bf16 MFMA flop/s, MI355X


def say(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def model_numbers(c):
    H, L, V = c["hidden_size"], c["num_hidden_layers"], c["vocab_size"]
    nq = c["num_attention_heads"] * c["head_dim"]
    nk = c["num_key_value_heads"] * c["head_dim"]
    F = c["intermediate_size"]
    layer_params = (nq + 2 * nk) * H + H * nq + 3 * H * F
    norm_params = 2 * H + 2 * c["head_dim"]
    head_params = V * H
    weight_bytes = L * (layer_params * 2 + norm_params * 4) + head_params * 2 + H * 4
    kv_bytes_per_token = 2 * nk * L * 2
    return dict(layer_params=layer_params, head_params=head_params, weight_bytes=weight_bytes,
                kv_bytes_per_token=kv_bytes_per_token)


def prefill_flops(c, T):
    n = model_numbers(c)
    L, nh, hd = c["num_hidden_layers"], c["num_attention_heads"], c["head_dim"]
    gemm = 2.0 * n["layer_params"] * L * T + 2.0 * n["head_params"]          # the head runs on one row
    attn = 2.0 * hd * T * (T + 1) * nh * L                                    # QK^T and PV over the causal half
    return gemm + attn


def fill(engine, rids, context, rng):
    """Give each request `context` cached tokens by real prefill steps."""
    import torch
    from tinyinfer_amd.engine import StepEntry
    V = engine.model.vocab_size
    for rid in rids:
        toks = rng.integers(0, V, size=context).tolist()
        engine.step([StepEntry(rid, toks, ())])
    torch.cuda.synchronize()


def measure_decode(engine, sampler, batch, steps, warmup, rng, tag):
    """tokens/s and ms/step of `steps` decode steps at `batch`, every request at CONTEXT tokens."""
    import torch
    from tinyinfer_amd.engine import StepEntry
    from tinyinfer_amd.sampling import SamplingParams
    rids = [f"{tag}{i}" for i in range(batch)]
    fill(engine, rids, CONTEXT, rng)
    greedy = [SamplingParams()] * batch
    nums = list(range(batch))
    last = rng.integers(0, engine.model.vocab_size, size=batch).tolist()

    def one_step(tokens):
        logits = engine.step_graph([StepEntry(r, [t], (0,)) for r, t in zip(rids, tokens)])
        return sampler.sample(logits, greedy, nums, nums)            # reads the ids back: a full sync

    for _ in range(warmup):
        last = one_step(last)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        last = one_step(last)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for r in rids:
        engine.release(r)
    return batch * steps / dt, dt / steps * 1e3


def measure_prefill(engine, rng, reps=5):
    import torch
    from tinyinfer_amd.engine import StepEntry
    V = engine.model.vocab_size
    times = []
    for i in range(reps + 2):
        toks = rng.integers(0, V, size=PREFILL_TOKENS).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = engine.step([StepEntry("prefill", toks, (PREFILL_TOKENS - 1,))])
        logits[0, :8].cpu()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.release("prefill")
    times = sorted(times[2:])                                       # the first two warm up
    return times[len(times) // 2]


def measure_mixed(engine, batch, portion, cached, rng, reps=8):
    """ms of a step that holds one decoded token of each of `batch` requests (CONTEXT tokens
    each) beside `portion` tokens of a prompt of which `cached` tokens are in the cache already:
    what the scheduler runs while a prompt arrives in portions.  Not a captured graph."""
    import torch
    from tinyinfer_amd.engine import StepEntry
    V = engine.model.vocab_size
    rids = [f"x{i}" for i in range(batch)]
    fill(engine, rids, CONTEXT, rng)
    times = []
    for i in range(reps + 3):
        if cached:
            engine.step([StepEntry("long", rng.integers(0, V, size=cached).tolist(), ())])
        entries = [StepEntry(r, [int(rng.integers(0, V))], (0,)) for r in rids]
        entries.append(StepEntry("long", rng.integers(0, V, size=portion).tolist(), (portion - 1,)))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = engine.step(entries)
        logits[0, :8].cpu()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.release("long")
    for r in rids:
        engine.release(r)
    times = sorted(times[3:])
    return times[len(times) // 2] * 1e3


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points")
    ap.add_argument("--only", choices=["all", "decode", "prefill", "mixed"], default="all",
                    help="measure one phase only (for profiles): the other's fields are null; "
                         "mixed: a step of --batch decoded tokens beside --portion tokens of a prompt, a line of its own")
    ap.add_argument("--portion", type=int, default=128, help="--only mixed: tokens of the prompt in the step")
    ap.add_argument("--cached", type=int, default=0, help="--only mixed: tokens of that prompt already in the cache")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not served (this engine runs on a single GPU)")
        return 2

    import numpy as np
    import torch
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.engine import Engine
    from tinyinfer_amd.sampling import Sampler

    cfg = dict(CONFIG)
    layers_full = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    rng = np.random.default_rng(0)
    biggest = max(args.batch, 1 if (args.no_points or args.only != "all") else 64)
    say("building the model (random weights on the device) ...")
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16", page_size=PAGE,
                                max_tokens=biggest * (CONTEXT + 512) + PREFILL_TOKENS + args.cached + args.portion,
                                max_requests=biggest + 1,
                                max_seq=MAX_SEQ)
    sampler = Sampler(engine.ops, engine.device)
    nums = model_numbers(cfg)

    if args.only == "mixed":
        say(f"a step of {args.batch} decoded tokens beside a portion of {args.portion} (after {args.cached} cached) ...")
        ms = measure_mixed(engine, args.batch, args.portion, args.cached, rng)
        print(json.dumps({"mixed": {"ms_per_step": round(ms, 3), "tokens": args.batch + args.portion,
                                    "decoded": args.batch, "portion": args.portion, "cached": args.cached,
                                    "decode_context": CONTEXT}}), flush=True)
        return 0
    p_s = tps = ms = None
    if args.only != "decode":
        say(f"prefill of {PREFILL_TOKENS} tokens ...")
        p_s = measure_prefill(engine, rng)
    if args.only != "prefill":
        say(f"decode at batch {args.batch} ...")
        tps, ms = measure_decode(engine, sampler, args.batch, args.steps, args.warmup, rng, "m")
    points = {}
    if not args.no_points and args.only == "all":
        for b, k in ((1, args.steps), (64, max(16, args.steps // 4))):
            say(f"decode at batch {b} ...")
            points[f"decode_b{b}"] = round(measure_decode(engine, sampler, b, k, max(4, args.warmup // 2), rng, f"p{b}_")[0], 1)

    ctx_mean = CONTEXT + args.warmup + args.steps / 2.0
    step_bytes = nums["weight_bytes"] + args.batch * ctx_mean * nums["kv_bytes_per_token"]
    achieved = step_bytes / (ms * 1e-3) if ms else None
    out = {
        "metric": f"decode tok/s @ batch {args.batch} (Qwen3-0.6B sizes, 2,048 cached tokens per request)",
        "value": None if tps is None else round(tps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": None if ms is None else round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": "Qwen3-0.6B sizes", "layers": cfg["num_hidden_layers"], "layers_in_config": layers_full,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"], "tied_head": True,
                   "global_batch": args.batch, "cached_tokens": CONTEXT, "seq_len": MAX_SEQ, "page_size": PAGE,
                   "prefill_tokens": PREFILL_TOKENS, "parallelism": "single GPU", "decode_graph": True},
        "prefill": None if p_s is None else
        {"value": round(PREFILL_TOKENS / p_s, 1), "tokens": PREFILL_TOKENS, "ms": round(p_s * 1e3, 3),
         "frac": round(prefill_flops(cfg, PREFILL_TOKENS) / p_s / PEAK_BF16, 4)},
        "roofline": None if achieved is None else
        {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
         "frac": round(achieved / PEAK_HBM, 4)},
        "points": points,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
