"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model 0.6b|1.7b|4b|8b|14b|32b] [--context N] [--prefill-tokens N]

The default run has the layer sizes of Qwen3-0.6B with random weights in
bfloat16: a batch of 8 requests, each holding 2,048 cached tokens (filled by
real prefill steps), decoded for K steps through the serving path (the step
function from a captured graph, greedy sampling on the device, the sampled
token fed back).  One JSON line goes to stdout: `value` is decoded tokens a
second at batch 8; `points` has batch 1 and 64; `prefill` a 2,048-token prompt in
one step; `roofline` the decode step's bytes (every weight once, the cache of
the live requests) over its time against 8 TB/s.  Beside the fractions of the
published peaks stand fractions of what this GPU delivers to a kernel that only
reads memory, and to matrix-core instructions on registers (csrc/measure.hip),
as the reference times its own kernels against the clock
(/root/reference/src/selftest.cpp:392-428).

`--model 8b` and `--model 32b` run the same with the sizes of Qwen3-8B and
Qwen3-32B.  `--kernel-times` adds a table of the decode step's calls, timed with
events (a line of its own on stderr).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import sys
import time

BASE = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", head_dim=128, vocab_size=151936,
            rope_theta=1000000.0, rms_norm_eps=1e-6, attention_bias=False, hidden_act="silu",
            max_position_embeddings=40960)
MODELS = {
    "0.6b": dict(BASE, num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                 intermediate_size=3072, tie_word_embeddings=True),
    "1.7b": dict(BASE, num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8,
                 intermediate_size=6144, tie_word_embeddings=True),
    "4b": dict(BASE, num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
               intermediate_size=9728, tie_word_embeddings=True),
    "8b": dict(BASE, num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
               intermediate_size=12288, tie_word_embeddings=False),
    "14b": dict(BASE, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=17408, tie_word_embeddings=False),
    "32b": dict(BASE, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                intermediate_size=25600, tie_word_embeddings=False),
}
NAMES = {"0.6b": "Qwen3-0.6B", "1.7b": "Qwen3-1.7B", "4b": "Qwen3-4B", "8b": "Qwen3-8B", "14b": "Qwen3-14B", "32b": "Qwen3-32B"}
MAX_SEQ = 4096            # context length a request may reach (more if --context asks for it)
PAGE = 16
PEAK_HBM = 8.0e12         # bytes/s, MI355X
PEAK_BF16 = 2.5e15        # dense bf16 MFMA flop/s, MI355X


def say(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def model_numbers(model):
    """What a step must read and compute, from what the model's parts declare (their tensors with roles, their
    cache needs), not from a formula of one architecture.  A decode step reads every matrix and vector of the
    layers and the head once (a head tied to the embedding reads the embedding's matrix) and one embedding row
    per token; per cached token it reads the keys and values of every cache layer."""
    seen = set()
    layer_params = head_params = vector_params = embed_row = 0
    attn = []                     # (heads, head_dim, window) of every mixer that attends over cached keys
    for part in model.parts():
        for name, need in part.tensors().items():
            n = 1
            for d in need.shape:
                n *= d
            if part.family == "embedding":
                embed_row = need.shape[-1]            # a row per token; the matrix counts where a head reads all of it
                continue
            if need.optional or name in seen:
                continue
            seen.add(name)
            if need.role != "matrix":
                vector_params += n
            elif part.family == "head":
                head_params += n
            else:
                layer_params += n
        need = part.cache_need()
        if need is not None and hasattr(need, "kv_heads") and "heads" in getattr(part, "params", {}):
            attn.append((part.params["heads"], need.head_dim, need.window))
    weight_bytes = (layer_params + head_params) * 2 + vector_params * 4 + embed_row * 2
    kv_bytes = lambda context: sum(2 * need.kv_heads * need.head_dim * 2 * n * min(context, need.window or context)      # noqa: E731
                                   for need, n in model.cache_groups if hasattr(need, "kv_heads"))
    return dict(layer_params=layer_params, head_params=head_params, weight_bytes=weight_bytes, kv_bytes=kv_bytes, attention=attn)


def prefill_flops(model, T):
    n = model_numbers(model)
    gemm = 2.0 * n["layer_params"] * T + 2.0 * n["head_params"]              # the head runs on one row
    attn = sum(2.0 * hd * T * (T + 1) * heads for heads, hd, _ in n["attention"])   # QK^T and PV over the causal half
    return gemm + attn


def measured_peaks():
    """(bytes/s of a kernel that only reads memory, flop/s of bfloat16 MFMAs on registers), the best of a few runs."""
    import torch
    from tinyinfer_amd import native
    from tinyinfer_amd.csrc import build
    native.ensure_kernels(["measure"])
    lib = ctypes.CDLL(build.find("measure"))
    lib.ti_measure_read.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    lib.ti_measure_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    n = 4 << 30
    buf = torch.empty(n, dtype=torch.uint8, device="cuda")
    buf.fill_(1)
    sink = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")

    def best(fn, reps=6):
        t = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            assert fn() == 0
            b.record()
            b.synchronize()
            t.append(a.elapsed_time(b) * 1e-3)
        return min(t[1:])
    units = torch.cuda.get_device_properties(0).multi_processor_count
    read = n / best(lambda: lib.ti_measure_read(buf.data_ptr(), n, sink.data_ptr(), units * 16, None))
    blocks, iters = units * 8, 4000
    mfma = blocks * 4 * iters * 4 * 32768 / best(lambda: lib.ti_measure_mfma(blocks, iters, sink.data_ptr(), None))
    del buf
    torch.cuda.empty_cache()
    return read, mfma


def decode_floor(engine, rids, last, nums, context, batch):
    """ms of a captured graph of kernels that only read memory, one for every call of a decode step in the step's own
    order, each reading as many bytes as that call has to (a product its weight, an attention the keys and values of
    the batch in one cache layer; everything else next to nothing): what a chain of so many dependent kernels over so
    many bytes takes on this GPU whatever the kernels compute.  The calls are the engine's own list for this step."""
    import re
    import torch
    from tinyinfer_amd import native
    from tinyinfer_amd.csrc import build
    from tinyinfer_amd.engine import StepEntry
    engine.ops.count_calls(True)
    engine.step([StepEntry(r, [t], (0,)) for r, t in zip(rids, last)])
    calls = engine.ops.timing_report()
    engine.ops.count_calls(False)
    layers = sum(n for need, n in engine.model.cache_groups if hasattr(need, "kv_heads"))
    kv_layer = nums["kv_bytes"](context) * batch // max(1, layers)
    sizes = []
    for c in calls:
        m = re.search(r"\* (\d+)x(\d+)", c["name"])
        per_call = int(m.group(1)) * int(m.group(2)) * 2 if m else kv_layer if c["name"].startswith("attention") else 4096
        sizes += [per_call] * c["calls"]
        if c["name"].startswith("attention") and "runs" in c["name"]:
            sizes += [4096] * c["calls"]              # the kernel that merges the runs of a context
    native.ensure_kernels(["measure"])
    lib = ctypes.CDLL(build.find("measure"))
    lib.ti_measure_read.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    total = sum(-(-b // 256) * 256 for b in sizes)
    buf = torch.empty(total + (1 << 20), dtype=torch.uint8, device="cuda")
    buf.fill_(1)
    sink = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")
    units = torch.cuda.get_device_properties(0).multi_processor_count
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            off = 0
            for b in sizes:
                b = -(-b // 256) * 256
                blocks = int(min(units * 8, max(1, b // 16384)))
                assert lib.ti_measure_read(buf.data_ptr() + off, b, sink.data_ptr(), blocks, stream.cuda_stream) == 0
                off += b
    best = None
    with torch.cuda.stream(stream):
        for _ in range(6):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()                 # (on the current stream)
            b.record()
            b.synchronize()
            best = a.elapsed_time(b) if best is None else min(best, a.elapsed_time(b))
    say(f"  a chain of {len(sizes)} kernels that only read {sum(sizes) / 1e6:.0f} MB: {best:.3f} ms")
    del graph, buf
    torch.cuda.empty_cache()
    return best, len(sizes)


def fill(engine, rids, context, rng, chunk=4096):
    """Give each request `context` cached tokens by real prefill steps."""
    import torch
    from tinyinfer_amd.engine import StepEntry
    V = engine.model.vocab_size
    for rid in rids:
        left = context
        while left > 0:
            n = min(left, chunk)
            engine.step([StepEntry(rid, rng.integers(0, V, size=n).tolist(), ())])
            left -= n
    torch.cuda.synchronize()


def measure_decode(engine, sampler, batch, steps, warmup, context, rng, tag, kernel_times=False, draw=None, floor=None):
    """tokens/s and ms/step of `steps` decode steps at `batch`, every request at `context` tokens.
    draw: (temperature, top_k, top_p) for the sampler, or None for the greedy choice."""
    import torch
    from tinyinfer_amd.engine import StepEntry, token_from_feedback
    from tinyinfer_amd.sampling import SamplingParams
    rids = [f"{tag}{i}" for i in range(batch)]
    fill(engine, rids, context, rng)
    greedy = [SamplingParams(draw[0], draw[1], draw[2], 1) if draw else SamplingParams()] * batch
    nums = list(range(batch))
    last = rng.integers(0, engine.model.vocab_size, size=batch).tolist()

    def one_step(tokens, graph=True):
        entries = [StepEntry(r, [t], (0,)) for r, t in zip(rids, tokens)]
        logits = engine.step_graph(entries) if graph else engine.step(entries)
        return sampler.sample(logits, greedy, nums, nums)            # reads the ids back: a full sync

    # As `run_requests` decodes: every step names its tokens by rows of the sampler's last call and is
    # launched before the ids of the step before it are read, so the device does not wait for the host.
    from_device = [StepEntry(r, [token_from_feedback(i)], (0,)) for i, r in enumerate(rids)]

    def steps_ahead(n, ticket):
        for _ in range(n):
            now = sampler.sample_async(engine.step_graph(from_device), greedy, nums, nums, feed=engine)
            sampler.collect(ticket)
            ticket = now
        return ticket

    for _ in range(min(2, warmup)):
        last = one_step(last)
    entries = [StepEntry(r, [t], (0,)) for r, t in zip(rids, last)]
    ticket = sampler.sample_async(engine.step_graph(entries), greedy, nums, nums, feed=engine)
    ticket = steps_ahead(max(0, warmup - 2), ticket)
    last = sampler.collect(ticket)
    entries = [StepEntry(r, [t], (0,)) for r, t in zip(rids, last)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ticket = sampler.sample_async(engine.step_graph(entries), greedy, nums, nums, feed=engine)
    ticket = steps_ahead(steps - 1, ticket)
    last = sampler.collect(ticket)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    if floor is not None:
        floor["ms"], floor["kernels"] = decode_floor(engine, rids, last, floor["nums"], context + warmup + steps, batch)
        last = one_step(last)
    table = None
    if kernel_times:
        one_step(last, graph=False)
        engine.ops.timing(True)
        for _ in range(4):
            last = one_step(last, graph=False)
        table = [dict(r, us=r["us"] / 4, calls=r["calls"] // 4) for r in engine.ops.timing_report()]
        engine.ops.timing(False)
    for r in rids:
        engine.release(r)
    return batch * steps / dt, dt / steps * 1e3, table


def measure_prefill(engine, rng, tokens, reps=5):
    import torch
    from tinyinfer_amd.engine import StepEntry
    V = engine.model.vocab_size
    times = []
    for i in range(reps + 2):
        toks = rng.integers(0, V, size=tokens).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = engine.step([StepEntry("prefill", toks, (tokens - 1,))])
        logits[0, :8].cpu()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.release("prefill")
    times = sorted(times[2:])                                       # the first two warm up
    return times[len(times) // 2]


def measure_mixed(engine, batch, portion, cached, context, rng, reps=8, graph=False):
    """ms of a step that holds one decoded token of each of `batch` requests (`context` tokens each)
    beside `portion` tokens of a prompt of which `cached` tokens are in the cache already: what the
    scheduler runs while a prompt arrives in portions.  graph: through `step_graph`, which replays a
    step's shape from a captured graph once it has come twice (generation with --cuda-graph).  Also
    the ms after which the host has handed the whole step to the GPU."""
    import torch
    from tinyinfer_amd.engine import StepEntry
    V = engine.model.vocab_size
    rids = [f"x{i}" for i in range(batch)]
    fill(engine, rids, context, rng)
    times, host = [], []
    for i in range(reps + 3):
        if cached:
            engine.step([StepEntry("long", rng.integers(0, V, size=cached).tolist(), ())])
        entries = [StepEntry(r, [int(rng.integers(0, V))], (0,)) for r in rids]
        entries.append(StepEntry("long", rng.integers(0, V, size=portion).tolist(), (portion - 1,)))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = (engine.step_graph if graph else engine.step)(entries)
        t1 = time.perf_counter()
        logits[0, :8].cpu()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        host.append(t1 - t0)
        engine.release("long")
    for r in rids:
        engine.release(r)
    times, host = sorted(times[3:]), sorted(host[3:])
    return times[len(times) // 2] * 1e3, host[len(host) // 2] * 1e3


def print_table(table, title):
    say(title)
    total = sum(r["us"] for r in table)
    for r in sorted(table, key=lambda r: -r["us"]):
        say(f"  {r['us']:9.1f} us  {r['calls']:4d} calls  {r['us'] / max(1, r['calls']):7.2f} us each  {r['name']}")
    say(f"  {total:9.1f} us  in all (events around every call; a graph replay leaves out the gaps between kernels)")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", choices=sorted(MODELS), default="0.6b", help="whose layer sizes the model has")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048, help="cached tokens each decoding request holds")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--temperature", type=float, default=0.0, help="decode draws its tokens at this temperature (0: greedy)")
    ap.add_argument("--top-k", type=int, default=0, help="with --temperature: the sampler's cut (0: its default, 512)")
    ap.add_argument("--top-p", type=float, default=1.0, help="with --temperature: the sampler's top-p")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points")
    ap.add_argument("--no-peaks", action="store_true", help="skip measuring the GPU's read bandwidth and MFMA rate")
    ap.add_argument("--kernel-times", action="store_true", help="a table of the decode step's calls, timed with events")
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

    cfg = dict(MODELS[args.model])
    layers_full = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    rng = np.random.default_rng(0)
    context, prefill_tokens = args.context, args.prefill_tokens
    max_seq = max(MAX_SEQ, context + args.warmup + args.steps + 64, prefill_tokens, args.cached + args.portion)
    biggest = max(args.batch, 1 if (args.no_points or args.only != "all") else 64)
    peaks = None
    if not args.no_peaks and args.only != "mixed":
        say("what the GPU delivers: a kernel that only reads, MFMAs on registers ...")
        peaks = measured_peaks()
        say(f"  read {peaks[0] / 1e9:.0f} GB/s, bf16 MFMA {peaks[1] / 1e12:.0f} TFLOP/s")
    say(f"building the model ({NAMES[args.model]} sizes, random weights on the device) ...")
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16", page_size=PAGE,
                                max_tokens=biggest * (context + 512) + prefill_tokens + args.cached + args.portion,
                                max_requests=biggest + 1, max_seq=max_seq)
    sampler = Sampler(engine.ops, engine.device)
    nums = model_numbers(engine.model)

    if args.only == "mixed":
        say(f"a step of {args.batch} decoded tokens beside a portion of {args.portion} (after {args.cached} cached) ...")
        ms, host_ms = measure_mixed(engine, args.batch, args.portion, args.cached, context, rng)
        g_ms, g_host = measure_mixed(engine, args.batch, args.portion, args.cached, context, rng, graph=True)
        print(json.dumps({"mixed": {"ms_per_step": round(ms, 3), "host_ms": round(host_ms, 3), "ms_from_graph": round(g_ms, 3),
                                    "host_ms_from_graph": round(g_host, 3), "tokens": args.batch + args.portion,
                                    "decoded": args.batch, "portion": args.portion, "cached": args.cached,
                                    "decode_context": context, "model": NAMES[args.model]}}), flush=True)
        return 0
    p_s = tps = ms = floor = None
    draw = (args.temperature, args.top_k, args.top_p) if args.temperature > 0 else None
    if args.only != "decode":
        say(f"prefill of {prefill_tokens} tokens ...")
        p_s = measure_prefill(engine, rng, prefill_tokens)
        if args.kernel_times:
            engine.ops.timing(True)
            measure_prefill(engine, rng, prefill_tokens, reps=2)
            table = [dict(r, us=r["us"] / 4, calls=r["calls"] // 4) for r in engine.ops.timing_report()]
            engine.ops.timing(False)
            print_table(table, f"a prefill step of {prefill_tokens} tokens, call by call:")
    if args.only != "prefill":
        say(f"decode at batch {args.batch} ...")
        floor = None if args.no_peaks else {"nums": nums}
        tps, ms, table = measure_decode(engine, sampler, args.batch, args.steps, args.warmup, context, rng, "m",
                                        args.kernel_times, draw, floor)
        if table:
            print_table(table, f"a decode step at batch {args.batch}, call by call (not from the graph):")
    points = {}
    if not args.no_points and args.only == "all":
        for b, k in ((1, args.steps), (64, max(16, args.steps // 4))):
            say(f"decode at batch {b} ...")
            points[f"decode_b{b}"] = round(measure_decode(engine, sampler, b, k, max(4, args.warmup // 2), context, rng,
                                                          f"p{b}_", draw=draw)[0], 1)

    ctx_mean = context + args.warmup + args.steps / 2.0
    step_bytes = nums["weight_bytes"] + args.batch * nums["kv_bytes"](ctx_mean)
    achieved = step_bytes / (ms * 1e-3) if ms else None
    roofline = prefill = None
    if achieved is not None:
        roofline = {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                    "frac": round(achieved / PEAK_HBM, 4)}
        if peaks:
            roofline.update(measured_read=round(peaks[0] / 1e9, 1), frac_of_measured=round(achieved / peaks[0], 4))
        if floor and floor.get("ms"):
            # a graph of as many kernels that only read as many bytes, in the step's order: the structure's own floor
            roofline.update(read_only_chain_ms=round(floor["ms"], 4), chain_kernels=floor["kernels"],
                            frac_of_read_only_chain=round(floor["ms"] / ms, 4))
    if p_s is not None:
        flops = prefill_flops(engine.model, prefill_tokens)
        prefill = {"value": round(prefill_tokens / p_s, 1), "tokens": prefill_tokens, "ms": round(p_s * 1e3, 3),
                   "frac": round(flops / p_s / PEAK_BF16, 4)}
        if peaks:
            prefill.update(measured_mfma_tflops=round(peaks[1] / 1e12, 1), frac_of_measured=round(flops / p_s / peaks[1], 4))
    out = {
        "metric": f"decode tok/s @ batch {args.batch} ({NAMES[args.model]} sizes, {context:,} cached tokens per request)",
        "value": None if tps is None else round(tps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": None if ms is None else round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": f"{NAMES[args.model]} sizes", "layers": cfg["num_hidden_layers"], "layers_in_config": layers_full,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "tied_head": bool(cfg["tie_word_embeddings"]),
                   "global_batch": args.batch, "cached_tokens": context, "seq_len": max_seq, "page_size": PAGE,
                   "prefill_tokens": prefill_tokens, "parallelism": "single GPU", "decode_graph": True,
                   "sampling": f"temperature {args.temperature} top-k {args.top_k or 512} top-p {args.top_p}" if draw else "greedy"},
        "prefill": prefill, "roofline": roofline, "points": points,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
