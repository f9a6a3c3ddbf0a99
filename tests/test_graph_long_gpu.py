"""Decode steps replayed from a graph that was captured for long sequences, and layers at the widths
of the two large benchmark configurations, against the plain implementation.

An engine whose longest sequence is 4,096 tokens captures its decode graph with the attention's
context cut into several runs (chosen for the longest sequence, frozen at capture: the partial
results' buffers, the number of runs) and replays it over rows of 3 to 2,100 cached tokens while
requests end and others take their pages.  The reference checks its graph against the eager step
the same way (/root/reference/src/inference.cu:297-341) and runs its kernels at real dimensions in
src/selftest.cpp:282-390,430-459."""
import numpy as np
import pytest

import traces
from helpers import CONFIGS, random_tokens
from test_engine_gpu import plain_logits, TOL

pytestmark = pytest.mark.gpu


def _decode_trace(requests, prompt, leaves, joins, n_before=20, n_after=20):
    """Prompts whole, one a step; `n_before` steps of one token of every live request (rows in changing
    order); `leaves` ends, `joins` is fed its prompt alone and takes the pages; `n_after` steps more."""
    live = [r for r in requests if r != joins]
    trace = [{"entries": [(r, requests[r][:prompt[r]], [prompt[r] - 1])], "end": []} for r in live]
    fed = dict(prompt)
    rows = {r: [prompt[r] - 1] for r in requests}

    def decode(k):
        order = live[k % len(live):] + live[:k % len(live)]
        trace.append({"entries": [(r, requests[r][fed[r]:fed[r] + 1], [0]) for r in order], "end": []})
        for r in order:
            rows[r].append(fed[r])
            fed[r] += 1
    for k in range(n_before):
        decode(k)
    trace[-1]["end"] = [leaves]
    live = [r for r in live if r != leaves] + [joins]
    trace.append({"entries": [(joins, requests[joins][:prompt[joins]], [prompt[joins] - 1])], "end": []})
    for k in range(n_after):
        decode(k)
    trace[-1]["end"] = list(live)
    return trace, rows, fed


def _replay(engine, trace, graph):
    from tinyinfer_amd.engine import StepEntry
    got = {}
    for step in trace:
        entries = [StepEntry(r, t, w) for r, t, w in step["entries"]]
        logits = (engine.step_graph(entries) if graph else engine.step(entries)).cpu().numpy().astype(np.float64)
        i = 0
        for r, _, w in step["entries"]:
            for _ in w:
                got.setdefault(r, []).append(logits[i])
                i += 1
        for r in step["end"]:
            engine.release(r)
        engine.cache.check()
    return {r: np.stack(v) for r, v in got.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["E", "D"])
def test_decode_graph_captured_for_long_sequences(model_folders, name, dtype):
    """Requests of 3, 17, 500 and 2,100 cached tokens decode together through `step_graph` on an engine whose
    longest sequence is 4,096: 20 steps, then the 17-token one ends, a newcomer takes its pages, 20 steps more.
    Every row is the plain model's; the same steps through `step` give the same bits in 32-bit and the same
    values within the bound in bfloat16 (the graph cuts the contexts into other runs than the eager step)."""
    import tinyinfer_amd as ti
    from tinyinfer_amd.ops import kernels as attention_bf16
    cfg = CONFIGS[name]
    folder = model_folders(name, "bfloat16", True)
    V = cfg["vocab_size"]
    prompt = {"a": 3, "b": 17, "c": 500, "d": 2100, "e": 30}
    total = {"a": 43, "b": 37, "c": 540, "d": 2140, "e": 50}
    requests = {r: random_tokens(n, V, 90 + i) for i, (r, n) in enumerate(total.items())}
    trace, rows, fed = _decode_trace(requests, prompt, leaves="b", joins="e")
    assert fed == total
    want, tol = plain_logits(folder, requests, dtype)
    if dtype == "float32":
        tol = TOL["float32"] * max(1.0, max(float(np.abs(want[r]).max()) for r in requests))
    pages = traces.max_pages(trace, 16)
    results = {}
    for graph in (True, False):
        engine = ti.Engine.from_folder(folder, dtype, page_size=16, num_pages=pages, max_requests=4, max_seq=4096)
        results[graph] = _replay(engine, trace, graph)
        assert not engine.cache.live_requests()
        if graph:
            assert 4 in engine.graph_keys(), engine.graph_keys()        # one decode graph for the batch of four
            for _, g in engine.cache.paged_groups():
                assert g.pool.taken_total > g.pool.num_pages or g.need.window    # the newcomer got pages that were used before
    if dtype == "bfloat16":
        # the launch the graph holds cuts a context into several runs and merges them: what the kernel tests
        # cover one launch at a time is wired into the engine here
        heads, kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
        assert attention_bf16.decode_splits(4, kv, heads, 4096, 2140, cfg["head_dim"]) > 1
    for r in requests:
        err = float(np.abs(results[True][r] - want[r][rows[r]]).max())
        print(f"\n[{name} {dtype} graph, max_seq 4096, request {r}] max |engine - plain| = {err:.3e} (allowed {tol:.3e})")
        assert err < tol, (r, err, tol)
        if dtype == "float32":
            assert np.array_equal(results[True][r], results[False][r]), r
        else:
            assert float(np.abs(results[True][r] - results[False][r]).max()) < tol, r


@pytest.mark.parametrize("dtype,theta", [("bfloat16", 123456.0), ("float32", 654321.0)])
def test_two_engines_do_not_share_what_a_graph_holds(tmp_path_factory, dtype, theta):
    """An engine with a short longest sequence captures a decode graph; then an engine with a longer one is
    built on a model with the same head size and rotation base (it needs a longer table of cosines and
    sines), and another one on the first engine's own model.  The table the first engine's graph reads stays
    where it is, and the graph replays to the same bits as before.  (A rotation base no other test uses, so
    that the first engine's table is its own and 256 positions long.)"""
    import tinyinfer_amd as ti
    from helpers import sharpen_folder
    from tinyinfer_amd.engine import StepEntry
    from tinyinfer_amd.weights import write_model_folder
    cfg = dict(CONFIGS["B"], rope_theta=theta, max_position_embeddings=8192)
    folder = str(tmp_path_factory.mktemp("two_engines"))
    write_model_folder(folder, cfg, seed=8, dtype="bfloat16")
    sharpen_folder(folder)
    toks = random_tokens(40, cfg["vocab_size"], 3)

    def run(engine, rid):
        out = [engine.step_graph([StepEntry(rid, toks[:20], [19])]).cpu().numpy().copy()]
        for t in toks[20:]:
            out.append(engine.step_graph([StepEntry(rid, [t], [0])]).cpu().numpy().copy())
        engine.release(rid)
        return np.concatenate(out)
    a = ti.Engine.from_folder(folder, dtype, page_size=16, max_tokens=256, max_requests=2, max_seq=256)
    pos = a.model.blocks[0].mixer.pos
    assert pos.table.shape[0] == 256
    table_before = pos.table.data_ptr()
    first = run(a, "x")
    assert 1 in a.graph_keys()
    b = ti.Engine.from_folder(folder, dtype, page_size=16, max_tokens=8192, max_requests=2, max_seq=8192)
    assert b.model.blocks[0].mixer.pos.table.shape[0] == 8192
    # a second engine on the first one's own model: the part now reads the longer table, the graph the old one
    c = ti.Engine(a.model, dtype, page_size=16, max_tokens=8192, max_requests=2, max_seq=8192)
    assert pos.table.shape[0] == 8192 and pos.table.data_ptr() != table_before
    junk = ti.native.torch().full((1 << 20,), 7.0, device="cuda")          # would land in memory that was given back
    again = run(a, "y")
    assert np.array_equal(first, again)
    if dtype == "float32":                      # (in bfloat16 a graph for longer sequences cuts the contexts into other runs)
        assert np.array_equal(first, run(c, "z"))
    del junk


WIDE = {
    # one layer with the widths of Qwen3-8B: 4,096 wide, 32 query heads on 8 kv heads, a feed-forward of 12,288
    "8B": dict(CONFIGS["F"], hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, intermediate_size=12288,
               vocab_size=1100, tie_word_embeddings=False),
    # one layer with the widths of Qwen3-32B: 5,120 wide, 64 query heads on 8 kv heads, a feed-forward of 25,600
    "32B": dict(CONFIGS["F"], hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, intermediate_size=25600,
                vocab_size=900, tie_word_embeddings=False),
}


@pytest.mark.parametrize("name", ["8B", "32B"])
def test_a_layer_at_the_widths_of_the_large_configurations(tmp_path_factory, name):
    """One layer at the widths of Qwen3-8B and of Qwen3-32B in bfloat16: a prompt of 2,048 tokens whole, then
    steps of 1, 8, 17, 64 and 136 rows (single tokens of up to 64 requests, the last one beside a portion of 73),
    against the plain model.  At these widths the products take branches no smaller model reaches (weights
    beyond 64 Mi elements, K split over workgroups for the stored projection, norms wider than 4,096)."""
    import tinyinfer_amd as ti
    from helpers import sharpen_folder
    from tinyinfer_amd.weights import write_model_folder
    cfg = WIDE[name]
    folder = str(tmp_path_factory.mktemp("wide" + name))
    write_model_folder(folder, cfg, seed=17, dtype="bfloat16")
    sharpen_folder(folder)
    V = cfg["vocab_size"]
    requests = {"a": random_tokens(2053, V, 61)}
    requests.update({f"s{i}": random_tokens(4 if i else 76, V, 100 + i) for i in range(63)})
    shorts = [f"s{i}" for i in range(63)]
    a = requests["a"]
    fed = {r: 0 for r in requests}
    rows = {r: [] for r in requests}

    def entry(r, n=1, want=None):
        want = [n - 1] if want is None else want
        e = (r, requests[r][fed[r]:fed[r] + n], want)
        rows[r] += [fed[r] + w for w in want]
        fed[r] += n
        return e
    trace = [{"entries": [entry("a", 2048, [0, 1000, 2047])], "end": []},
             {"entries": [entry("a")], "end": []},                                            # 1 row
             {"entries": [entry("a")] + [entry(r) for r in shorts[:7]], "end": []},            # 8 rows
             {"entries": [entry("a")] + [entry(r) for r in shorts[:16]], "end": []},           # 17 rows
             {"entries": [entry("a")] + [entry(r) for r in shorts], "end": []},                # 64 rows
             {"entries": [entry("a")] + [entry("s0", 73, [0, 72])] + [entry(r) for r in shorts[1:]], "end": []}]  # 136 rows
    assert [sum(len(t) for _, t, _ in s["entries"]) for s in trace] == [2048, 1, 8, 17, 64, 136]
    trace[-1]["end"] = list(requests)
    requests = {r: t[:fed[r]] for r, t in requests.items()}
    want, tol = plain_logits(folder, requests, "bfloat16")
    engine = ti.Engine.from_folder(folder, "bfloat16", page_size=16, num_pages=traces.max_pages(trace, 16), max_requests=64,
                                   max_seq=2112)
    engine.ops.count_calls(True)
    got = _replay(engine, trace, False)
    calls = [c["name"] for c in engine.ops.timing_report()]
    worst = 0.0
    for r in requests:
        err = float(np.abs(got[r] - want[r][rows[r]]).max())
        worst = max(worst, err)
        assert err < tol, (r, err, tol)
    print(f"\n[{name} widths, bfloat16] max |engine - plain| = {worst:.3e} (allowed {tol:.3e})")
    # the kernels these widths are tested for did run: matrix-core products (none fell to the generic kernel),
    # the norm inside the product for the small steps, the projection that finishes its heads for the prompt, the
    # decode attention that prepares its own query
    def ran(start, tag):
        return any(c.startswith(start) and tag in c for c in calls)
    assert ran("linear.add 2048x", "[mfma]") and ran("linear.swiglu 2048x", "[mfma]") and ran("linear.add 64x", "[mfma"), calls
    # (the norm goes into the product of a step of few rows up to a width of 4,096 and under a weight of 64 Mi elements)
    assert ran("norm+linear.store 8x", "[fused]") or cfg["hidden_size"] > 4096, [c for c in calls if " 8x" in c]
    assert ran("qkv_prepared 2048x", "[fused]"), calls
    assert ran("attention.decode_prepared rows=64", "[fused"), calls
    assert not any("[generic]" in c for c in calls), calls
